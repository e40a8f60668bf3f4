"""The C-ABI library loads and exports exactly what include/emm_kv.h declares (no GPU needed)."""
import ctypes
import os
import re

import pytest

from elasticmm_amd import _lib, library_path

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "emm_kv.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(emm_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for name in ("emm_kv_pack", "emm_kv_unpack", "emm_copy_blocks", "emm_reshape_and_cache",
                 "emm_reshape_and_cache_fp8", "emm_kv_unpack_dequant_fp8", "emm_concat_rows", "emm_last_error"):
        assert name in syms


def test_library_exports_every_declared_symbol():
    assert os.path.exists(library_path()), "libemm_kv.so has not been built"
    lib = ctypes.CDLL(library_path())
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in emm_kv.h but not exported"


def test_hooks_exist_only_in_the_hooks_build():
    """The product library carries no benchmark switch or probe: those live in libemm_kv_hooks.so, which
    exports the whole product ABI next to them (so a benchmark can route its calls through it)."""
    from elasticmm_amd.build import hooks_library_path

    hooks_header = open(os.path.join(ROOT, "elasticmm_amd", "csrc", "emm_kv_hooks.h")).read()
    hooks_header = re.sub(r"/\*.*?\*/", "", hooks_header, flags=re.S)
    hook_syms = sorted(set(re.findall(r"\b(emm_hook_[a-z0-9_]+)\s*\(", hooks_header)))
    assert hook_syms == sorted(_lib.HOOK_SIGNATURES) and len(hook_syms) >= 3
    product = ctypes.CDLL(library_path())
    for name in hook_syms + ["emm_set_move_variant"]:
        assert not hasattr(product, name), f"{name} must not be exported by the product library"
    assert os.path.exists(hooks_library_path()), "libemm_kv_hooks.so has not been built"
    hooks = ctypes.CDLL(hooks_library_path())
    for name in hook_syms + declared_symbols():
        assert hasattr(hooks, name), f"{name} missing from the hooks build"
    # nothing in the package reaches for the hooks build on its own
    pkg = os.path.join(ROOT, "elasticmm_amd")
    for fn in os.listdir(pkg):
        if fn.endswith(".py") and fn not in ("_lib.py", "build.py"):
            text = open(os.path.join(pkg, fn)).read()
            assert "hooks" not in text, f"{fn} refers to the hooks build"


def test_binding_table_matches_header():
    assert sorted(_lib.SIGNATURES) == declared_symbols()
    text = open(HEADER).read()
    assert int(re.search(r"#define EMM_MAX_LAYERS (\d+)", text).group(1)) == _lib.EMM_MAX_LAYERS
    assert int(re.search(r"#define EMM_MAX_SEGMENTS (\d+)", text).group(1)) == _lib.EMM_MAX_SEGMENTS
    assert int(re.search(r"#define EMM_KV_ABI_VERSION (\d+)", text).group(1)) == _lib.EMM_KV_ABI_VERSION


def test_load_and_argument_errors_without_gpu():
    """Argument validation happens before any HIP call, so it can be exercised on a CPU-only host."""
    lib = _lib.load()
    assert lib.emm_abi_version() == _lib.EMM_KV_ABI_VERSION
    table = _lib.ptr_table([0x1000])
    rc = lib.emm_kv_pack(table, 200, 2, 4, 64, 0x1000, 1, 0x1000, None)
    assert rc == -1 and b"num_layers" in lib.emm_last_error()
    rc = lib.emm_kv_pack(table, 1, 2, 4, -64, 0x1000, 1, 0x1000, None)
    assert rc == -1 and b"negative" in lib.emm_last_error()
    rc = lib.emm_kv_pack(table, 1, 2, 4, 64, None, 1, 0x1000, None)
    assert rc == -1 and b"null" in lib.emm_last_error()
    # empty work is a no-op that never reaches the device
    assert lib.emm_kv_pack(table, 1, 2, 4, 64, None, 0, None, None) == 0
    assert lib.emm_concat_rows(None, None, 0, None, 0, None) == 0
    assert lib.emm_concat_rows(None, None, 1000, None, 0, None) == -1
    with pytest.raises(_lib.EmmError, match="emm_concat_rows"):
        _lib.check(-1, "emm_concat_rows")
    rc = lib.emm_reshape_and_cache(0x1000, 0x1000, 0x1000, 0x1000, 0x1000, 4, 64, 32, 64, 16, None)
    assert rc == -1 and b"stride" in lib.emm_last_error()
    rc = lib.emm_kv_unpack_dequant_fp8(table, 1, 4, 24, 0x1000, 1, 0x1000, 0x1000, 0x1000, 0, None)
    assert rc == -1 and b"multiples of 16" in lib.emm_last_error()


def test_argument_errors_of_the_layout_variants_without_gpu():
    lib = _lib.load()
    P = 0x1000
    # paged-attention layout: head_size must be a multiple of x = 16 / cache element bytes
    rc = lib.emm_reshape_and_cache_paged(P, P, P, P, P, 4, 2, 20, 16, 8, 40, 40, 0, 2, None, None, None)
    assert rc == -1 and b"multiple of x" in lib.emm_last_error()
    rc = lib.emm_reshape_and_cache_paged(P, P, P, P, P, 4, 2, 32, 16, 8, 64, 64, 0, 3, None, None, None)
    assert rc == -1 and b"cache_elem_bytes" in lib.emm_last_error()
    rc = lib.emm_reshape_and_cache_paged(P, P, P, P, P, 4, 2, 32, 16, 8, 64, 64, 0, 1, None, None, None)
    assert rc == -1 and b"scale" in lib.emm_last_error()
    rc = lib.emm_reshape_and_cache_paged(P, P, P, P + 8, P, 4, 2, 32, 16, 8, 64, 64, 0, 2, None, None, None)
    assert rc == -1 and b"16-byte aligned" in lib.emm_last_error()
    rc = lib.emm_reshape_and_cache_paged(P, P, P, P, P, 4, 2, 32, 0, 8, 64, 64, 0, 2, None, None, None)
    assert rc == -1 and b"negative size" in lib.emm_last_error()
    assert lib.emm_reshape_and_cache_paged(P, P, P, P, P, 0, 2, 32, 16, 8, 64, 64, 0, 2, None, None, None) == 0
    t = _lib.ptr_table([P])
    rc = lib.emm_reshape_and_cache_paged_layers(t, t, t, t, 97, P, 4, 2, 32, 16, 8, 64, 64, 0, 2, None, None, None)
    assert rc == -1 and b"num_layers" in lib.emm_last_error()
    # strided flash layout: strides must cover a head row
    rc = lib.emm_reshape_and_cache_strided(t, t, t, t, 1, P, 4, 2, 64, 16, 8, 128, 128, 4096, 32, 64, None)
    assert rc == -1 and b"stride smaller than a head row" in lib.emm_last_error()
    rc = lib.emm_reshape_and_cache_strided(t, t, t, t, 1, P, 4, 2, 64, 16, 8, 100, 128, 4096, 128, 64, None)
    assert rc == -1 and b"token stride" in lib.emm_last_error()
    assert lib.emm_reshape_and_cache_strided(t, t, t, t, 0, P, 4, 2, 64, 16, 8, 128, 128, 4096, 128, 64, None) == 0


def test_last_error_is_kept_per_thread():
    """Two host threads that fail in different ways each read their own message (the text lives in
    thread-local storage; the transfer manager calls the library from a thread of its own)."""
    import threading

    lib = _lib.load()
    table = _lib.ptr_table([0x1000])
    seen, start = {}, threading.Barrier(2)

    def worker(name, layers, want):
        start.wait()
        for _ in range(200):
            rc = lib.emm_kv_pack(table, layers, 2, 4, 64 if layers == 200 else -64, 0x1000, 1, 0x1000, None)
            msg = lib.emm_last_error()
            if rc != -1 or want not in msg:
                seen[name] = msg
                return
        seen[name] = b"ok"

    a = threading.Thread(target=worker, args=("a", 200, b"num_layers"))
    b = threading.Thread(target=worker, args=("b", 1, b"negative"))
    a.start(), b.start()
    a.join(), b.join()
    assert seen == {"a": b"ok", "b": b"ok"}
    assert lib.emm_kv_pack(table, 1, 2, 4, 64, None, 0, None, None) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "library_path", lambda: str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()
