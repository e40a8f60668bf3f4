"""ctypes binding of libemm_kv.so (the C ABI of include/emm_kv.h).

There is no fallback: if the shared object is missing or an entry point fails,
the caller gets an exception.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p, POINTER

from .build import hooks_library_path, library_path

EMM_KV_ABI_VERSION = 3
EMM_MAX_LAYERS = 96
EMM_MAX_SEGMENTS = 128
EMM_MAX_INLINE_IDS = 512
EMM_DTYPE_BF16 = 0
EMM_DTYPE_F16 = 1
EMM_FP8_SATURATE = 0x100

_P = c_void_p
_PP = POINTER(c_void_p)
_I64P = POINTER(c_int64)

# name -> (restype, argtypes); mirrors include/emm_kv.h one to one
SIGNATURES = {
    "emm_last_error": (c_char_p, []),
    "emm_abi_version": (c_int, []),
    "emm_kv_pack": (c_int, [_PP, c_int, c_int, c_int64, c_int64, _P, c_int64, _P, _P]),
    "emm_kv_unpack": (c_int, [_PP, c_int, c_int, c_int64, c_int64, _P, c_int64, _P, _P]),
    "emm_kv_pack_host_ids": (c_int, [_PP, c_int, c_int, c_int64, c_int64, _P, c_int64, _P, _P]),
    "emm_kv_unpack_host_ids": (c_int, [_PP, c_int, c_int, c_int64, c_int64, _P, c_int64, _P, _P]),
    "emm_copy_blocks": (c_int, [_PP, c_int, c_int, c_int64, c_int64, _P, c_int64, _P]),
    "emm_kv_migrate": (c_int, [_PP, c_int64, _PP, c_int64, c_int, c_int, c_int64, _P, _P, c_int64, _P]),
    "emm_kv_unpack_dequant_fp8": (c_int, [_PP, c_int, c_int64, c_int64, _P, c_int64, _P, _P, _P, c_int, _P]),
    "emm_reshape_and_cache": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, _P]),
    "emm_reshape_and_cache_layers": (c_int, [_PP, _PP, _PP, _PP, c_int, _P, c_int64, c_int64, c_int64, c_int64,
                                             c_int64, _P]),
    "emm_reshape_and_cache_fp8": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64,
                                          _P, _P, c_int, _P]),
    "emm_reshape_and_cache_fp8_layers": (c_int, [_PP, _PP, _PP, _PP, c_int, _P, c_int64, c_int64, c_int64,
                                                 c_int64, c_int64, _P, _P, c_int, _P]),
    "emm_reshape_and_cache_strided": (c_int, [_PP, _PP, _PP, _PP, c_int, _P, c_int64, c_int, c_int64, c_int, c_int64,
                                              c_int64, c_int64, c_int64, c_int64, c_int64, _P]),
    "emm_reshape_and_cache_strided_fp8": (c_int, [_PP, _PP, _PP, _PP, c_int, _P, c_int64, c_int, c_int64, c_int, c_int64,
                                                  c_int64, c_int64, c_int64, c_int64, c_int64, _P, _P, c_int, _P]),
    "emm_reshape_and_cache_paged": (c_int, [_P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int64, c_int64,
                                            c_int64, c_int, c_int, _P, _P, _P]),
    "emm_reshape_and_cache_paged_layers": (c_int, [_PP, _PP, _PP, _PP, c_int, _P, c_int64, c_int, c_int, c_int,
                                                   c_int64, c_int64, c_int64, c_int, c_int, _P, _P, _P]),
    "emm_concat_rows": (c_int, [_PP, _I64P, c_int, _P, c_int64, _P]),
    "emm_stream_copy": (c_int, [_P, _P, c_int64, _P]),
}

# libemm_kv_hooks.so only (csrc/emm_kv_hooks.h): benchmark / test hooks, absent from the product library
HOOK_SIGNATURES = {
    "emm_hook_set_move_variant": (c_int, [c_int]),
    "emm_hook_probe": (c_int, [c_int, _PP, c_int, c_int, c_int64, c_int64, _P, c_int64, _P, _P, _P]),
    "emm_hook_pack_variant": (c_int, [c_int, _PP, c_int, c_int, c_int64, c_int64, _P, c_int64, _P, _P]),
    "emm_hook_empty_launch": (c_int, [_P]),
    "emm_hook_fp8_quotient_sweep": (c_int, [c_int, c_int, ctypes.c_uint32, ctypes.c_uint32, _P, _P]),
}
EMM_PROBE_SEQ_READ, EMM_PROBE_SEQ_WRITE, EMM_PROBE_GATHER_READ, EMM_PROBE_SCATTER_WRITE = 0, 1, 2, 3
EMM_PROBE_GATHER_READ_COMPUTED_IDS, EMM_PROBE_PACK_COMPUTED_IDS, EMM_PROBE_PACK = 4, 5, 6
EMM_PROBE_PACK_NOTHING_FETCHED = 7
EMM_PACK_VARIANTS = {"two_tiles_per_workgroup": 1, "whole_chunk_per_workgroup": 2, "lds_dma_4KiB_one_wave": 3,
                     "lds_dma_16KiB_four_waves": 4, "lds_dma_8KiB_one_wave": 5, "loader_storer_split": 6}

_lib = None
_hooks = None


class EmmError(RuntimeError):
    """An entry point of libemm_kv.so returned a non-zero code."""


def load() -> ctypes.CDLL:
    """Load libemm_kv.so once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            f"{path} is missing: the HIP library has not been built "
            "(run `python -m elasticmm_amd.build`). There is no CPU fallback.")
    # torch carries its own copy of the HIP runtime and exports its symbols globally. Streams and device pointers
    # come from torch, so the library has to bind to that copy: torch is loaded before the library is.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = res
        fn.argtypes = args
    ver = lib.emm_abi_version()
    if ver != EMM_KV_ABI_VERSION:
        raise RuntimeError(f"libemm_kv.so ABI version {ver}, expected {EMM_KV_ABI_VERSION}")
    _lib = lib
    return lib


def load_hooks() -> ctypes.CDLL:
    """Load libemm_kv_hooks.so (bench.py and tests only): the product ABI plus the hooks."""
    global _hooks
    if _hooks is not None:
        return _hooks
    path = hooks_library_path()
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing (run `python -m elasticmm_amd.build`)")
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    lib = ctypes.CDLL(path)
    for name, (res, args) in {**SIGNATURES, **HOOK_SIGNATURES}.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _hooks = lib
    return lib


def use_hooks_build() -> ctypes.CDLL:
    """Route every later call of this process through libemm_kv_hooks.so, so that a benchmark can switch
    launch variants (``emm_hook_set_move_variant``). Never called by the package itself."""
    global _lib
    _lib = load_hooks()
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().emm_last_error().decode("utf-8", "replace")
        raise EmmError(f"{what} failed with code {rc}: {msg}")


def ptr_table(ptrs) -> ctypes.Array:
    """A host array of device pointers for the `layer_ptrs`-style arguments."""
    return (c_void_p * len(ptrs))(*ptrs)
