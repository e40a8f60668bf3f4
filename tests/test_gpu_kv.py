"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle.

Bit-exact everywhere (byte moves and the fp8 cast alike): pools, transfer buffers
and caches are compared as raw bit patterns. Small and medium shapes are compared
with the oracle in full; the full-size shapes (two 51 GiB pools) are checked through
size-independent properties (every moved block equals its source, everything
else keeps its canary) evaluated on the device with torch indexing as a second,
independent implementation.
"""
import json
import os

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import kv_oracle as orc  # noqa: E402  (test infrastructure)
from elasticmm_amd import _lib, cache_ops, kv_ops, pool_transfer  # noqa: E402
from elasticmm_amd.kv_ops import PoolView  # noqa: E402
from elasticmm_amd.block_manager import BlockLocation, BlockManager  # noqa: E402
from elasticmm_amd.worker import KVWorker, LoopbackLink  # noqa: E402

DEV = "cuda:0"


@pytest.fixture(scope="module", autouse=True)
def _need_gpu():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    _lib.load()
    yield
    torch.cuda.synchronize()


def say(msg):
    print(msg, flush=True)


def raw(t: torch.Tensor) -> np.ndarray:
    """Bit pattern of a tensor as a flat uint8 numpy array (host)."""
    return t.detach().contiguous().cpu().reshape(-1).view(torch.uint8).numpy()


def same_bits(a: torch.Tensor, b) -> bool:
    """True if a and b hold the same bytes; otherwise fails with a short summary of the
    first differences (never prints the tensors)."""
    bb = raw(b) if isinstance(b, torch.Tensor) else np.ascontiguousarray(b).reshape(-1).view(np.uint8)
    aa = raw(a)
    if aa.size != bb.size:
        pytest.fail(f"size differs: {aa.size} vs {bb.size} bytes", pytrace=False)
    bad = np.nonzero(aa != bb)[0]
    if bad.size:
        first = bad[:8]
        pytest.fail(f"{bad.size} of {aa.size} bytes differ; first at byte offsets {first.tolist()}: "
                    f"got {aa[first].tolist()} want {bb[first].tolist()}", pytrace=True)
    return True


def cpu_pool(L, NB, bs, H, D, dtype, seed, scale=1.0, fill=None):
    g = torch.Generator().manual_seed(seed)
    out = []
    for _ in range(L):
        if fill is not None:
            out.append(torch.full((2, NB, bs, H, D), fill, dtype=dtype))
        else:
            out.append((torch.randn((2, NB, bs, H, D), generator=g) * scale).to(dtype))
    return out


def to_dev(pool, monolithic=False):
    if monolithic:
        return list(torch.stack(pool, 0).to(DEV).unbind(0))
    return [p.to(DEV) for p in pool]


# ------------------------------------------------------------------ config 1
def test_cfg1_pack_unpack_bitwise():
    say("cfg1: L4 [2,1024,16,8,128] fp16, 32 blocks, seeds 0/1")
    L, NB, bs, H, D = 4, 1024, 16, 8, 128
    src_c = cpu_pool(L, NB, bs, H, D, torch.float16, 0)
    dst_c = cpu_pool(L, NB, bs, H, D, torch.float16, 0, fill=-3.0)
    src_idx = torch.randperm(NB, generator=torch.Generator().manual_seed(0))[:32].tolist()
    dst_idx = torch.randperm(NB, generator=torch.Generator().manual_seed(1))[:32].tolist()
    src_g, dst_g = to_dev(src_c), to_dev(dst_c)
    sw, dw = KVWorker(device=DEV), KVWorker(device=DEV)
    sw.bind_kv_cache(src_g)
    dw.bind_kv_cache(dst_g)
    buf = sw.extract_kv_blocks(src_idx)
    assert buf.shape == (L, 2, 32, bs, H, D) and buf.dtype == torch.float16 and buf.is_contiguous()
    assert buf.numel() * 2 == 8 << 20
    want = orc.ref_extract_kv_blocks(src_c, src_idx)
    assert same_bits(buf, want)
    assert same_bits(buf, orc.c_kv_pack(src_c, src_idx))
    dw.write_kv_blocks(dst_idx, buf)
    orc.ref_write_kv_blocks(dst_c, dst_idx, want)
    for l in range(L):
        assert same_bits(dst_g[l], dst_c[l]), f"layer {l}"
        assert same_bits(src_g[l], src_c[l])
    assert sw.get_kv_cache_layout() == {"num_layers": 4, "block_size": 16, "num_heads": 8, "head_size": 128,
                                        "dtype": "float16"}


def test_golden_fixture_through_the_gpu(golden_dir):
    z = np.load(os.path.join(golden_dir, "kv_small.npz"))

    def t16(a, dt=torch.float16):
        return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(dt).to(DEV)

    src = [t16(a) for a in z["src"]]
    pool = PoolView(src)
    packed = kv_ops.kv_pack(pool, z["src_idx"].tolist())
    assert same_bits(packed, z["packed"])
    dst = [torch.full_like(p, -7.0) for p in src]
    kv_ops.kv_unpack(PoolView(dst), z["dst_idx"].tolist(), packed)
    assert same_bits(torch.stack(dst), z["dst_after"])
    NB, bs, H, D = z["key_cache_after"].shape
    kc = torch.full((NB, bs, H, D), 3.0, dtype=torch.float16, device=DEV)
    vc = torch.full((NB, bs, H, D), 5.0, dtype=torch.float16, device=DEV)
    cache_ops.reshape_and_cache_flash(t16(z["key"]), t16(z["value"]), kc, vc, torch.from_numpy(z["slots"]).to(DEV))
    assert same_bits(kc, z["key_cache_after"]) and same_bits(vc, z["value_cache_after"])
    cb = [p.clone() for p in src]
    cache_ops.copy_blocks(cb, torch.from_numpy(z["mapping"]).to(DEV))
    assert same_bits(torch.stack(cb), z["copy_after"])
    segs = [t16(z[f"seg{i}"], torch.bfloat16) for i in range(3)]
    assert same_bits(kv_ops.concat_rows(segs), z["cat"])


# ------------------------------------------------------------------ shapes / edge cases
@pytest.mark.parametrize("dtype,bs,H,D,desc", [
    (torch.bfloat16, 16, 4, 128, "16 KiB chunk, one full tile"),
    (torch.float16, 16, 8, 128, "32 KiB chunk, two tiles"),
    (torch.bfloat16, 16, 5, 128, "20 KiB chunk, tail tile"),
    (torch.bfloat16, 2, 1, 64, "256 B chunk, smaller than a tile"),
    (torch.float16, 1, 1, 3, "6 B chunk, 2-byte lanes"),
    (torch.float32, 1, 1, 5, "20 B chunk, 4-byte lanes"),
    (torch.uint8, 1, 1, 7, "7 B chunk, byte lanes"),
    (torch.float32, 16, 2, 64, "fp32 pool"),
])
@pytest.mark.parametrize("monolithic", [False, True])
def test_pack_unpack_shapes(dtype, bs, H, D, desc, monolithic):
    say(f"shape case: {desc} monolithic={monolithic}")
    L, NB, n = 3, 37, 9
    g = torch.Generator().manual_seed(21)
    if dtype == torch.uint8:
        src_c = [torch.randint(0, 255, (2, NB, bs, H, D), generator=g, dtype=torch.uint8) for _ in range(L)]
        dst_c = [torch.full((2, NB, bs, H, D), 0xAB, dtype=torch.uint8) for _ in range(L)]
    else:
        src_c = cpu_pool(L, NB, bs, H, D, dtype, 21)
        dst_c = cpu_pool(L, NB, bs, H, D, dtype, 0, fill=-5.0)
    si = torch.randperm(NB, generator=g)[:n].tolist()
    di = torch.randperm(NB, generator=g)[:n].tolist()
    src_g, dst_g = to_dev(src_c, monolithic), to_dev(dst_c, monolithic)
    buf = kv_ops.kv_pack(PoolView(src_g), si)
    assert same_bits(buf, orc.c_kv_pack(src_c, si))
    kv_ops.kv_unpack(PoolView(dst_g), di, buf)
    orc.c_kv_unpack(dst_c, di, raw(buf))
    for l in range(L):
        assert same_bits(dst_g[l], dst_c[l])


def test_empty_and_single_block():
    src_c = cpu_pool(2, 8, 4, 2, 16, torch.bfloat16, 5)
    src_g = to_dev(src_c)
    pool = PoolView(src_g)
    e = kv_ops.kv_pack(pool, [])
    assert e.shape == (2, 2, 0, 4, 2, 16)
    kv_ops.kv_unpack(pool, [], e)
    kv_ops.copy_blocks(pool, torch.zeros((0, 2), dtype=torch.long, device=DEV))
    one = kv_ops.kv_pack(pool, [7])
    assert same_bits(one, orc.ref_extract_kv_blocks(src_c, [7]))
    k = torch.zeros((0, 2, 16), dtype=torch.bfloat16, device=DEV)
    kv_ops.reshape_and_cache(k, k, src_g[0][0], src_g[0][1], torch.zeros((0,), dtype=torch.long, device=DEV))
    for l in range(2):
        assert same_bits(src_g[l], src_c[l])


def test_list_indices_follow_torch_rules_on_gpu():
    src_c = cpu_pool(1, 6, 2, 1, 8, torch.float16, 6)
    pool = PoolView(to_dev(src_c))
    got = kv_ops.kv_pack(pool, [-1, 0, -6])
    assert same_bits(got, orc.ref_extract_kv_blocks(src_c, [-1, 0, -6]))
    with pytest.raises(IndexError):
        kv_ops.kv_pack(pool, [6])


def test_device_indices_padding_and_out_of_range_are_skipped():
    src_c = cpu_pool(2, 6, 2, 1, 8, torch.float16, 7)
    pool = PoolView(to_dev(src_c))
    idx = torch.tensor([4, -1, 99, 0], dtype=torch.long, device=DEV)
    out = torch.full((2, 2, 4, 2, 1, 8), 1.25, dtype=torch.float16, device=DEV)
    kv_ops.kv_pack(pool, idx, out=out)
    want = torch.full((2, 2, 4, 2, 1, 8), 1.25, dtype=torch.float16)
    ref = orc.ref_extract_kv_blocks(src_c, [4, 0])
    want[:, :, 0] = ref[:, :, 0]
    want[:, :, 3] = ref[:, :, 1]
    assert same_bits(out, want)
    dst_c = cpu_pool(2, 6, 2, 1, 8, torch.float16, 0, fill=2.0)
    dst_g = to_dev(dst_c)
    kv_ops.kv_unpack(PoolView(dst_g), idx, out)
    orc.c_kv_unpack(dst_c, [4, -1, 99, 0], raw(out))
    for l in range(2):
        assert same_bits(dst_g[l], dst_c[l])


def test_strict_mode_catches_bad_device_ids_and_the_default_skips_them():
    """A device-resident block table with ids outside the pool: by default the kernels skip those ids and touch
    nothing else (neighbouring blocks keep their canary); with strict=True the caller gets IndexError before
    anything is launched — on kv_pack, kv_unpack, kv_migrate, copy_blocks and through the worker's switch."""
    L, NB, bs, H, D = 2, 24, 16, 2, 64
    src_c = cpu_pool(L, NB, bs, H, D, torch.bfloat16, seed=3)
    src = PoolView(to_dev(src_c))
    good = torch.tensor([5, 0, 23, 7], device=DEV)
    for bad_id in (-1, NB, 10 ** 9):
        bad = torch.tensor([5, bad_id, 23, 7], device=DEV)
        # default: skipped, the other rows are right
        buf = kv_ops.kv_pack(src, bad)
        want = orc.ref_extract_kv_blocks(src_c, [5, 0, 23, 7])
        for j in (0, 2, 3):
            assert same_bits(buf[:, :, j], want[:, :, j])
        dst_c = cpu_pool(L, NB, bs, H, D, torch.bfloat16, seed=4, fill=7.0)
        dst = PoolView(to_dev(dst_c))
        kv_ops.kv_unpack(dst, bad, kv_ops.kv_pack(src, good))
        for l in range(L):
            for j, b in enumerate([5, 0, 23, 7]):
                if j != 1:
                    dst_c[l][:, b] = want[l][:, j]
            assert same_bits(dst.layers[l], dst_c[l]), "a skipped id touched a neighbour"
        # strict: IndexError, nothing written
        for call in (lambda: kv_ops.kv_pack(src, bad, strict=True),
                     lambda: kv_ops.kv_unpack(dst, bad, buf, strict=True),
                     lambda: kv_ops.kv_migrate(src, bad, dst, good, strict=True),
                     lambda: kv_ops.kv_migrate(src, good, dst, bad, strict=True),
                     lambda: kv_ops.copy_blocks(dst, torch.stack([good, bad], 1).contiguous(), strict=True),
                     lambda: cache_ops.copy_blocks(dst.layers, torch.stack([bad, good], 1).contiguous(), strict=True)):
            with pytest.raises(IndexError, match="out of bounds"):
                call()
        torch.cuda.synchronize()
        for l in range(L):
            assert same_bits(dst.layers[l], dst_c[l]), "a strict call that raised wrote something"
    # good tables pass in strict mode and give the same result
    assert same_bits(kv_ops.kv_pack(src, good, strict=True), orc.ref_extract_kv_blocks(src_c, [5, 0, 23, 7]))
    w = KVWorker(0, DEV, bs)
    w.bind_kv_cache(src.layers)
    w.strict_device_tables = True
    with pytest.raises(IndexError):
        w.extract_kv_blocks(torch.tensor([1, NB], device=DEV))
    assert same_bits(w.extract_kv_blocks(good), orc.ref_extract_kv_blocks(src_c, [5, 0, 23, 7]))


def test_two_host_threads_on_two_streams_at_once():
    """The library is re-entrant: two host threads, each with its own stream and its own pair of pools, issue 200
    rounds of pack / unpack / append at the same time (the pattern of the reference's side streams,
    elasticmm/engine/v0/worker.py:496-516). Every round's transfer buffer and both final pools are compared with
    the oracle replaying the same sequence; thread 0 also makes an invalid call now and then, and thread 1's
    error string (per host thread) must stay empty throughout."""
    import threading

    lib = _lib.load()
    L, NB, bs, H, D, rounds = 3, 96, 16, 2, 64, 200
    results = {}

    def work(tid):
        try:
            g = torch.Generator().manual_seed(100 + tid)
            src_c = cpu_pool(L, NB, bs, H, D, torch.bfloat16, seed=50 + tid)
            dst_c = cpu_pool(L, NB, bs, H, D, torch.bfloat16, seed=60 + tid, fill=float(tid + 1))
            stream = torch.cuda.Stream()
            bufs, errors = [], []
            with torch.cuda.stream(stream):
                src_g, dst_g = to_dev(src_c), to_dev(dst_c)
                sp, dp = PoolView(src_g), PoolView(dst_g)
                plan = []
                for r in range(rounds):
                    n = int(torch.randint(1, 9, (1,), generator=g))
                    si = torch.randperm(NB, generator=g)[:n]
                    di = torch.randperm(NB, generator=g)[:n]
                    T = int(torch.randint(1, 40, (1,), generator=g))
                    slots = torch.randperm(NB * bs, generator=g)[:T]
                    slots[::7] = -1
                    key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
                    value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
                    l = r % L
                    plan.append((si, di, slots, key, value, l))
                    # tables alternate between host lists and device tensors (both entry-point families)
                    buf = kv_ops.kv_pack(sp, si.tolist() if r & 1 else si.to(DEV))
                    kv_ops.kv_unpack(dp, di.to(DEV) if r & 1 else di.tolist(), buf)
                    cache_ops.reshape_and_cache_flash(key.to(DEV), value.to(DEV), src_g[l][0], src_g[l][1],
                                                      slots.to(DEV), "auto")
                    bufs.append(buf)
                    if tid == 0 and r % 50 == 0:
                        assert lib.emm_kv_pack(None, -1, 2, NB, 64, None, 1, None, None) != 0
                    errors.append(lib.emm_last_error())
            stream.synchronize()
            # the oracle replays the sequence
            for r, (si, di, slots, key, value, l) in enumerate(plan):
                want = orc.ref_extract_kv_blocks(src_c, si.tolist())
                assert same_bits(bufs[r], want), f"thread {tid} round {r}: pack"
                orc.ref_write_kv_blocks(dst_c, di.tolist(), want)
                orc.c_reshape_and_cache(key, value, src_c[l][0], src_c[l][1], slots)
            for l in range(L):
                assert same_bits(src_g[l], src_c[l]) and same_bits(dst_g[l], dst_c[l]), f"thread {tid} layer {l}"
            results[tid] = errors
        except BaseException as e:  # noqa: BLE001 - reported by the main thread
            results[tid] = e

    threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    for tid in (0, 1):
        if isinstance(results[tid], BaseException):
            raise results[tid]
    assert all(e == b"" for e in results[1]), "thread 1 saw an error string it did not cause"
    assert any(b"num_layers" in e for e in results[0]), "thread 0's invalid calls left no message"


def test_pack_variants_of_the_hooks_build_give_the_pack():
    """The alternative kernel shapes kept in the hooks build for re-measuring (two and four tiles per workgroup,
    loads straight into LDS, loader / storer waves) must compute the same pack, skipped ids included."""
    hooks = _lib.load_hooks()
    for H, n in ((4, 37), (8, 130), (4, 1)):          # 16 KiB and 32 KiB chunks
        L, NB, bs, D = 3, 200, 16, 128
        pool_c = cpu_pool(L, NB, bs, H, D, torch.bfloat16, seed=H + n)
        pool = PoolView(to_dev(pool_c))
        g = torch.Generator().manual_seed(n)
        ids = torch.randperm(NB, generator=g)[:n].clone()
        if n > 4:
            ids[3], ids[n - 2] = -1, NB + 5
        ids_g = ids.to(DEV)
        want = torch.full(pool.packed_shape(n), 7.0, dtype=torch.bfloat16, device=DEV)
        kv_ops.kv_pack(pool, ids_g, out=want)
        table = _lib.ptr_table(pool.ptrs)
        for name, code in _lib.EMM_PACK_VARIANTS.items():
            say(f"pack variant {name}: chunk {pool.chunk_bytes} bytes, {n} blocks")
            got = torch.full(pool.packed_shape(n), 7.0, dtype=torch.bfloat16, device=DEV)
            rc = hooks.emm_hook_pack_variant(code, table, L, 2, NB, pool.chunk_bytes, ids_g.data_ptr(), n, got.data_ptr(),
                                             torch.cuda.current_stream().cuda_stream)
            assert rc == 0, hooks.emm_last_error()
            assert same_bits(got, want.cpu()), name


def test_more_layers_than_one_argument_block():
    L = _lib.EMM_MAX_LAYERS + 5
    src_c = cpu_pool(L, 5, 1, 1, 8, torch.float16, 8)
    src_g = to_dev(src_c)
    buf = kv_ops.kv_pack(PoolView(src_g), [3, 1])
    assert same_bits(buf, orc.ref_extract_kv_blocks(src_c, [3, 1]))
    dst_g = [torch.zeros_like(p) for p in src_g]
    kv_ops.kv_unpack(PoolView(dst_g), [0, 4], buf)
    dst_c = [torch.zeros_like(p) for p in src_c]
    orc.ref_write_kv_blocks(dst_c, [0, 4], orc.ref_extract_kv_blocks(src_c, [3, 1]))
    assert same_bits(torch.stack(dst_g), torch.stack(dst_c))
    kv_ops.kv_migrate(PoolView(src_g), [2], PoolView(dst_g), [1])
    assert same_bits(torch.stack(dst_g)[:, :, 1], torch.stack(src_c)[:, :, 2])


# ------------------------------------------------------------------ copy_blocks / migrate
def test_copy_blocks_against_oracle():
    L, NB = 5, 64
    base = cpu_pool(L, NB, 16, 4, 128, torch.bfloat16, 9, scale=0.5)
    g = torch.Generator().manual_seed(9)
    perm = torch.randperm(NB, generator=g)
    mapping = torch.stack([perm[:20], perm[20:40]], 1).contiguous()
    dev = to_dev(base)
    cache_ops.copy_blocks(dev, mapping.to(DEV))
    want = [p.clone() for p in base]
    orc.c_copy_blocks(want, mapping.numpy())
    ref = [p.clone() for p in base]
    orc.ref_copy_blocks(ref, mapping)
    for l in range(L):
        assert same_bits(dev[l], want[l]) and same_bits(dev[l], ref[l])
        assert same_bits(dev[l][:, perm[:20].to(DEV)], base[l][:, perm[:20]])  # sources unchanged
    # list-of-pairs form goes through the same path
    dev2 = to_dev(base)
    kv_ops.copy_blocks(PoolView(dev2), mapping.tolist())
    assert same_bits(torch.stack(dev2), torch.stack(want))


def test_copy_blocks_with_split_key_and_value_caches():
    """The operator-level call shape: per-layer key caches and value caches of the paged-attention layout
    (different trailing shapes, equal bytes per block), checked against the C restatement applied to the same
    bytes viewed as [2, NB, chunk] pools and against torch's indexing."""
    for dtype, L, NB, H, D, bs in [(torch.bfloat16, 3, 50, 4, 128, 16), (torch.uint8, 2, 40, 2, 64, 16),
                                   (torch.float16, 100, 12, 1, 32, 8)]:  # 200 planes: more than one argument block
        x = 16 // torch.empty((), dtype=dtype).element_size()
        g = torch.Generator().manual_seed(NB + L)
        kcs = [torch.randint(0, 250, (NB, H, D // x, bs, x), generator=g).to(dtype) for _ in range(L)]
        vcs = [torch.randint(0, 250, (NB, H, D, bs), generator=g).to(dtype) for _ in range(L)]
        perm = torch.randperm(NB, generator=g)
        n = NB // 3
        mapping = torch.stack([perm[:n], perm[n:2 * n]], 1).contiguous()
        k_g, v_g = to_dev(kcs), to_dev(vcs)
        cache_ops.copy_blocks(k_g, v_g, mapping.to(DEV))
        pools = [torch.stack([kcs[l].reshape(NB, -1), vcs[l].reshape(NB, -1)]) for l in range(L)]
        orc.c_copy_blocks(pools, mapping.numpy())
        for l in range(L):
            assert same_bits(k_g[l], pools[l][0]) and same_bits(v_g[l], pools[l][1]), f"layer {l}"
            want_k = kcs[l].clone()
            want_k[mapping[:, 1]] = kcs[l][mapping[:, 0]]
            assert same_bits(k_g[l], want_k)
    cache_ops.copy_blocks([], [], mapping.to(DEV))  # nothing to do
    with pytest.raises(ValueError, match="differ in length"):
        cache_ops.copy_blocks(k_g, v_g[:-1], mapping.to(DEV))


def test_cache_ops_swap_blocks_between_gpu_and_pinned_host():
    """vLLM's swap_blocks for one layer: GPU -> page-locked host -> another GPU cache, K and V per launch;
    the pairs arrive as a CPU tensor (vLLM's form) or as a list."""
    NBg, NBc, bs, H, D = 30, 20, 16, 4, 128
    g = torch.Generator().manual_seed(77)
    gpu_c = torch.randn((2, NBg, bs, H, D), generator=g).to(torch.bfloat16)
    gpu = gpu_c.to(DEV)
    cpu = torch.zeros((2, NBc, bs, H, D), dtype=torch.bfloat16).pin_memory()
    out_pairs = torch.stack([torch.randperm(NBg, generator=g)[:12], torch.randperm(NBc, generator=g)[:12]], 1)
    cache_ops.swap_blocks(gpu, cpu, out_pairs)
    torch.cuda.synchronize()
    want_cpu = torch.zeros_like(cpu)
    want_cpu[:, out_pairs[:, 1]] = gpu_c[:, out_pairs[:, 0]]
    assert same_bits(cpu, want_cpu)
    back = torch.full((2, NBg, bs, H, D), 7.0, dtype=torch.bfloat16, device=DEV)
    in_pairs = torch.stack([out_pairs[:, 1], torch.randperm(NBg, generator=g)[:12]], 1)
    cache_ops.swap_blocks(cpu, back, in_pairs.tolist())
    want_back = torch.full((2, NBg, bs, H, D), 7.0, dtype=torch.bfloat16)
    want_back[:, in_pairs[:, 1]] = want_cpu[:, in_pairs[:, 0]]
    assert same_bits(back, want_back)
    gpu2 = torch.zeros_like(gpu)
    cache_ops.swap_blocks(gpu, gpu2, out_pairs[:, [0, 0]].contiguous())  # device to device, same ids
    want2 = torch.zeros_like(gpu_c)
    want2[:, out_pairs[:, 0]] = gpu_c[:, out_pairs[:, 0]]
    assert same_bits(gpu2, want2)
    cache_ops.swap_blocks(gpu, gpu2, torch.empty((0, 2), dtype=torch.long))  # nothing to do
    with pytest.raises(ValueError, match="GPU memory"):
        cache_ops.swap_blocks(cpu, cpu, out_pairs)


def test_migrate_equals_pack_then_unpack():
    L, NBs, NBd = 4, 40, 24
    src_c = cpu_pool(L, NBs, 16, 4, 128, torch.bfloat16, 10)
    g = torch.Generator().manual_seed(10)
    si = torch.randperm(NBs, generator=g)[:12].tolist()
    di = torch.randperm(NBd, generator=g)[:12].tolist()
    src_g = to_dev(src_c)
    a = [torch.full((2, NBd, 16, 4, 128), 1.0, dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    b = [t.clone() for t in a]
    kv_ops.kv_migrate(PoolView(src_g), si, PoolView(a), di)
    kv_ops.kv_unpack(PoolView(b), di, kv_ops.kv_pack(PoolView(src_g), si))
    assert same_bits(torch.stack(a), torch.stack(b))
    with pytest.raises(ValueError, match="Block count mismatch"):
        kv_ops.kv_migrate(PoolView(src_g), si, PoolView(a), di[:-1])


def test_block_moves_seeded_sweep_of_shapes():
    """Thirty seeded draws of (dtype, block size, heads, head size, layers, pool size, table length, table as a list
    or on the device, one allocation or one per layer): pack, unpack, migrate and copy_blocks against the C
    restatement. Table lengths straddle the 512 ids that one launch carries in its argument block."""
    g = torch.Generator().manual_seed(977)
    pick = lambda xs: xs[int(torch.randint(len(xs), (1,), generator=g))]  # noqa: E731
    for case in range(30):
        dtype = pick([torch.bfloat16, torch.float16, torch.float32, torch.uint8])
        bs, H, D = pick([1, 2, 8, 16, 32]), pick([1, 2, 3, 5, 8]), pick([3, 7, 16, 40, 64, 128])
        L = pick([1, 2, 7, 33])
        n = pick([1, 2, 31, 511, 512, 513, 700])
        if bs * H * D * L * n > (48 << 20):
            n = 31
        NB = n + pick([1, 5, 64])
        as_list, mono = pick([True, False]), pick([True, False])
        say(f"block-move sweep {case}: {dtype} bs={bs} H={H} D={D} L={L} NB={NB} n={n} list={as_list} mono={mono}")
        if dtype == torch.uint8:
            src_c = [torch.randint(0, 255, (2, NB, bs, H, D), generator=g, dtype=torch.uint8) for _ in range(L)]
        else:
            src_c = [torch.randint(-30000, 30000, (2, NB, bs, H, D), generator=g).to(dtype) for _ in range(L)]
        dst_c = [torch.zeros_like(t) for t in src_c]
        si_t, di_t = torch.randperm(NB, generator=g)[:n], torch.randperm(NB, generator=g)[:n]
        si, di = (si_t.tolist(), di_t.tolist()) if as_list else (si_t.to(DEV), di_t.to(DEV))
        src_g, dst_g, mig_g = to_dev(src_c, mono), to_dev(dst_c, mono), to_dev(dst_c, mono)
        buf = kv_ops.kv_pack(PoolView(src_g), si)
        assert same_bits(buf, orc.c_kv_pack(src_c, si_t.tolist())), f"pack, case {case}"
        kv_ops.kv_unpack(PoolView(dst_g), di, buf)
        orc.c_kv_unpack(dst_c, di_t.tolist(), raw(buf))
        assert same_bits(torch.stack(dst_g), torch.stack(dst_c)), f"unpack, case {case}"
        kv_ops.kv_migrate(PoolView(src_g), si, PoolView(mig_g), di)
        assert same_bits(torch.stack(mig_g), torch.stack(dst_c)), f"migrate, case {case}"
        half = n // 2
        if half:
            perm = torch.randperm(NB, generator=g)
            mapping = torch.stack([perm[:half], perm[half:2 * half]], 1).contiguous()
            if as_list:
                kv_ops.copy_blocks(PoolView(src_g), mapping.tolist())
            else:
                cache_ops.copy_blocks(src_g, mapping.to(DEV))
            orc.c_copy_blocks(src_c, mapping.numpy())
            assert same_bits(torch.stack(src_g), torch.stack(src_c)), f"copy_blocks, case {case}"


@pytest.mark.parametrize("bs,H,D,desc", [
    (16, 1, 128, "4 KiB chunks: one tile"), (16, 2, 128, "8 KiB: two tiles"), (16, 3, 128, "12 KiB: three tiles"),
    (16, 4, 128, "16 KiB"), (16, 5, 128, "20 KiB: five tiles"), (16, 6, 128, "24 KiB: six tiles"),
    (11, 8, 128, "22 KiB: six tiles, the last one partly filled"), (16, 8, 128, "32 KiB"), (16, 9, 128, "36 KiB: nine tiles"),
    (16, 10, 128, "40 KiB: ten tiles"), (16, 40, 128, "160 KiB: forty tiles"),
])
def test_block_moves_of_a_hundred_blocks_over_tiles_per_chunk(bs, H, D, desc):
    """Tables of 96 blocks and more choose a tile-to-XCD mapping by the number of tiles per chunk (pairs of tiles for
    an even count, whole chunks for pool-to-pool moves of 8 tiles and more or of an odd count, none otherwise); the
    mapping works on windows of 8 blocks, so the table lengths here leave 4, 3 and 0 blocks past the last window."""
    L = 3
    g = torch.Generator().manual_seed(bs * 1000 + H)
    for n in (100, 131, 96):
        NB = n + 40
        say(f"block moves, {desc}, {n} blocks")
        src_c = [torch.randint(-30000, 30000, (2, NB, bs, H, D), generator=g).to(torch.bfloat16) for _ in range(L)]
        dst_c = [torch.zeros_like(t) for t in src_c]
        si_t, di_t = torch.randperm(NB, generator=g)[:n], torch.randperm(NB, generator=g)[:n]
        src_g, dst_g, dst2_g, mig_g = to_dev(src_c), to_dev(dst_c), to_dev(dst_c), to_dev(dst_c)
        want = orc.c_kv_pack(src_c, si_t.tolist())
        buf = kv_ops.kv_pack(PoolView(src_g), si_t.to(DEV))
        assert same_bits(buf, want), "pack, device table"
        assert same_bits(kv_ops.kv_pack(PoolView(src_g), si_t.tolist()), want), "pack, list"
        kv_ops.kv_unpack(PoolView(dst_g), di_t.to(DEV), buf)
        kv_ops.kv_unpack(PoolView(dst2_g), di_t.tolist(), buf)
        orc.c_kv_unpack(dst_c, di_t.tolist(), raw(buf))
        assert same_bits(torch.stack(dst_g), torch.stack(dst_c)), "unpack, device table"
        assert same_bits(torch.stack(dst2_g), torch.stack(dst_c)), "unpack, list"
        kv_ops.kv_migrate(PoolView(src_g), si_t.to(DEV), PoolView(mig_g), di_t.to(DEV))
        assert same_bits(torch.stack(mig_g), torch.stack(dst_c)), "migrate"
        perm = torch.randperm(NB, generator=g)
        mapping = torch.stack([perm[:n // 2 + 20], perm[n // 2 + 20:2 * (n // 2 + 20)]], 1).contiguous()
        cache_ops.copy_blocks(src_g, mapping.to(DEV))
        orc.c_copy_blocks(src_c, mapping.numpy())
        assert same_bits(torch.stack(src_g), torch.stack(src_c)), "copy_blocks"


@pytest.mark.parametrize("H,NB,n", [(4, 10400, 100), (4, 14000, 131), (40, 1100, 100), (6, 7000, 99), (2, 25000, 120)])
def test_pack_of_a_short_table_from_large_planes(H, NB, n):
    """A pack pairs its tiles per XCD only when the table is short against the plane it indexes (blocks * 2 MiB up to
    1.25 x the plane's bytes): planes of 160 MB and more here, with 4, 40, 6 and 2 tiles per chunk (a power of two
    and not)."""
    bs, D = 16, 128
    assert n * (2 << 20) <= 1.25 * NB * bs * H * D * 2
    g = torch.Generator().manual_seed(NB + n)
    src_c = [torch.randint(-30000, 30000, (2, NB, bs, H, D), generator=g, dtype=torch.int16).view(torch.bfloat16)]
    si = torch.randperm(NB, generator=g)[:n]
    src_g = to_dev(src_c)
    want = orc.c_kv_pack(src_c, si.tolist())
    assert same_bits(kv_ops.kv_pack(PoolView(src_g), si.to(DEV)), want), "device table"
    assert same_bits(kv_ops.kv_pack(PoolView(src_g), si.tolist()), want), "list"


@pytest.mark.parametrize("bs,H,D,n", [(16, 8, 128, 100), (16, 4, 128, 131), (16, 5, 128, 100), (16, 1, 128, 97),
                                      (16, 8, 128, 1100)])
def test_dequant_unpack_of_a_hundred_blocks_over_tiles_per_chunk(bs, H, D, n):
    L, NB = 2, n + 30
    g = torch.Generator().manual_seed(n + H)
    packed = torch.randint(0, 0x78, (L, 2, n, bs, H, D), generator=g, dtype=torch.uint8)  # finite positive e4m3
    packed[:, :, ::3] |= 0x80
    ks, vs = torch.tensor([0.03, 0.4]), torch.tensor([0.9, 0.011])
    di = torch.randperm(NB, generator=g)[:n]
    for dt in (torch.bfloat16, torch.float16):
        dq_g = [torch.full((2, NB, bs, H, D), 9.0, dtype=dt, device=DEV) for _ in range(L)]
        dq_c = [torch.full((2, NB, bs, H, D), 9.0, dtype=dt) for _ in range(L)]
        kv_ops.kv_unpack_dequant_fp8(PoolView(dq_g), di.to(DEV), packed.to(DEV), ks, vs)
        orc.c_unpack_dequant_fp8(dq_c, di.tolist(), raw(packed), ks.numpy(), vs.numpy())
        assert same_bits(torch.stack(dq_g), torch.stack(dq_c)), str(dt)


# ------------------------------------------------------------------ legacy pools
def test_monolithic_6d_pool_and_vision_pool():
    L, NB, bs, H, D = 3, 20, 16, 2, 64
    g = torch.Generator().manual_seed(11)
    pool6 = torch.randn((L, 2, NB, bs, H, D), generator=g).to(torch.float16)
    si, di = [7, 0, 19, 3], [1, 2, 18, 5]
    flat = pool_transfer.gather_kv_blocks(pool6.to(DEV), si)
    assert flat.dim() == 1 and same_bits(flat, orc.ref_pool6d_gather(pool6, si))
    dst_c = torch.zeros_like(pool6)
    dst_g = dst_c.to(DEV)
    kv_data = pool_transfer.scatter_kv_blocks(dst_g, di, flat)
    assert kv_data.shape == (L, 2, 4, bs, H, D)
    orc.ref_pool6d_scatter(dst_c, di, orc.ref_pool6d_gather(pool6, si))
    assert same_bits(dst_g, dst_c)
    ve = torch.randn((12, 9, 48), generator=g).to(torch.bfloat16)
    vf = pool_transfer.gather_vision_blocks(ve.to(DEV), [5, 11, 0])
    assert same_bits(vf, orc.ref_vision_gather(ve, [5, 11, 0]))
    ve_dst_c = torch.zeros_like(ve)
    ve_dst_g = ve_dst_c.to(DEV)
    pool_transfer.scatter_vision_blocks(ve_dst_g, [2, 3, 4], vf)
    orc.ref_vision_scatter(ve_dst_c, [2, 3, 4], orc.ref_vision_gather(ve, [5, 11, 0]))
    assert same_bits(ve_dst_g, ve_dst_c)


def test_pool_transfer_manager_sender_and_receiver_halves():
    """The legacy manager's two halves over the loopback link: what the receiver's pool holds afterwards is the
    torch statement of the reference's stack / per-block assignment, for the 6-D KV pool and the vision pool."""
    import asyncio
    from elasticmm_amd.worker import LoopbackLink

    L, NB, bs, H, D = 3, 20, 16, 2, 64
    g = torch.Generator().manual_seed(12)
    pool6 = torch.randn((L, 2, NB, bs, H, D), generator=g).to(torch.bfloat16)
    si, di = [7, 0, 19, 3, 11], [1, 2, 18, 5, 0]
    link = LoopbackLink(2)
    sender, receiver = pool_transfer.PoolTransferManager(link), pool_transfer.PoolTransferManager(link)
    with pytest.raises(ValueError, match="Group 'g' not found"):
        sender.transfer_kv_cache_blocks_sync("g", 0, 1, pool6.to(DEV), si, di, True)
    sender.create_transfer_group("g", 0, 2)
    receiver.create_transfer_group("g", 1, 2)
    src_g, dst_c = pool6.to(DEV), torch.zeros_like(pool6)
    dst_g = dst_c.to(DEV)
    assert asyncio.run(sender.transfer_kv_cache_blocks("g", 0, 1, src_g, si, di, True)) is None
    kv_data = asyncio.run(receiver.transfer_kv_cache_blocks("g", 0, 1, dst_g, si, di, False))
    assert kv_data.shape == (L, 2, len(si), bs, H, D)
    orc.ref_pool6d_scatter(dst_c, di, orc.ref_pool6d_gather(pool6, si))
    assert same_bits(dst_g, dst_c) and same_bits(src_g, pool6)
    st = sender.get_stats()
    assert st["total_transfers"] == 1 and st["total_bytes_transferred"] == kv_data.numel() * 2 and st["num_groups"] == 1
    ve = torch.randn((12, 9, 48), generator=g).to(torch.float16)
    ve_dst_c = torch.zeros_like(ve)
    ve_dst_g = ve_dst_c.to(DEV)
    assert sender.transfer_vision_embeddings_sync("g", 0, 1, ve.to(DEV), [5, 11, 0], [2, 3, 4], True) is None
    got = receiver.transfer_vision_embeddings_sync("g", 0, 1, ve_dst_g, [5, 11, 0], [2, 3, 4], False)
    assert got.shape == (3, 9, 48)
    orc.ref_vision_scatter(ve_dst_c, [2, 3, 4], orc.ref_vision_gather(ve, [5, 11, 0]))
    assert same_bits(ve_dst_g, ve_dst_c)
    # a message of the wrong type is refused before anything is written
    sender.transfer_vision_embeddings_sync("g", 0, 1, ve.to(DEV), [1], [1], True)
    with pytest.raises(ValueError, match="differs from the pool's"):
        receiver.transfer_vision_embeddings_sync("g", 0, 1, ve_dst_g.to(torch.bfloat16), [1], [1], False)


# ------------------------------------------------------------------ append
def make_slots(num_slots, T, seed, pad_frac=0.05):
    g = torch.Generator().manual_seed(seed)
    slots = torch.randperm(num_slots, generator=g)[:T].clone()
    pad = torch.rand(T, generator=g) < pad_frac
    slots[pad] = -1
    return slots


def test_cfg3_append_reduced_pool():
    say("cfg3 shape: T=8448 [T,4,128] bf16, 5% padded slots; pool reduced to 2048 blocks, 2 layers")
    NB, bs, H, D, T, L = 2048, 16, 4, 128, 8448, 2
    slots = make_slots(NB * bs, T, 3)
    assert (slots < 0).sum() > 300
    g = torch.Generator().manual_seed(3)
    pool_c = cpu_pool(L, NB, bs, H, D, torch.bfloat16, 0, fill=7.0)
    pool_g = to_dev(pool_c)
    slots_g = slots.to(DEV)
    for l in range(L):
        key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
        value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
        cache_ops.reshape_and_cache_flash(key.to(DEV), value.to(DEV), pool_g[l][0], pool_g[l][1], slots_g, "auto")
        orc.c_reshape_and_cache(key, value, pool_c[l][0], pool_c[l][1], slots)
        assert same_bits(pool_g[l], pool_c[l]), f"layer {l}"
    ref = cpu_pool(1, NB, bs, H, D, torch.bfloat16, 0, fill=7.0)[0]
    orc.ref_reshape_and_cache_flash(key, value, ref[0], ref[1], slots)
    assert same_bits(pool_g[L - 1], ref)


@pytest.mark.parametrize("T", [1, 3, 1536, 1537, 2051, 6144, 6145, 6147])
def test_append_token_counts_around_the_wave_shape_thresholds(T):
    """The per-layer append picks 1, 2 or 4 token rows per wave from the token count: both sides of each
    threshold, and counts that leave the last wave partly empty."""
    NB, bs, H, D = 512, 16, 4, 128
    slots = make_slots(NB * bs, T, T, pad_frac=0.05)
    g = torch.Generator().manual_seed(T)
    key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    pool_c = cpu_pool(1, NB, bs, H, D, torch.bfloat16, 0, fill=3.0)
    pool_g = to_dev(pool_c)
    cache_ops.reshape_and_cache_flash(key.to(DEV), value.to(DEV), pool_g[0][0], pool_g[0][1], slots.to(DEV), "auto")
    orc.c_reshape_and_cache(key, value, pool_c[0][0], pool_c[0][1], slots)
    assert same_bits(pool_g[0], pool_c[0])


def test_append_strided_tokens_odd_rows_and_layers_variant():
    NB, bs, H, D, T, L = 16, 4, 3, 40, 37, 3  # 240-byte rows (16-B lanes), T not a multiple of 16
    g = torch.Generator().manual_seed(13)
    qkv = torch.randn((L, T, 3 * H * D), generator=g).to(torch.float16)
    slots = make_slots(NB * bs, T, 13, pad_frac=0.2)
    pool_c = cpu_pool(L, NB, bs, H, D, torch.float16, 0, fill=1.0)
    pool_g = to_dev(pool_c)
    qkv_g = qkv.to(DEV)
    keys = [qkv_g[l, :, H * D:2 * H * D].view(T, H, D) for l in range(L)]       # strided views
    values = [qkv_g[l, :, 2 * H * D:].view(T, H, D) for l in range(L)]
    assert not keys[0].is_contiguous()
    cache_ops.reshape_and_cache_flash_layers(keys, values, pool_g, slots.to(DEV))
    for l in range(L):
        k = qkv[l, :, H * D:2 * H * D].reshape(T, H, D).contiguous()
        v = qkv[l, :, 2 * H * D:].reshape(T, H, D).contiguous()
        orc.c_reshape_and_cache(k, v, pool_c[l][0], pool_c[l][1], slots)
        assert same_bits(pool_g[l], pool_c[l])
    # per-layer call on a strided view, narrow rows (6 bytes -> 2-byte lanes)
    kc = torch.zeros((4, 2, 1, 3), dtype=torch.float16, device=DEV)
    vc = torch.zeros_like(kc)
    x = torch.randn((5, 2, 3), generator=g).to(torch.float16)
    xs = x.to(DEV)[:, 1:2, :]
    sl = torch.tensor([7, -1, 0, 3, 5])
    cache_ops.reshape_and_cache_flash(xs, xs, kc, vc, sl.to(DEV))
    kcc = torch.zeros((4, 2, 1, 3), dtype=torch.float16)
    vcc = torch.zeros_like(kcc)
    orc.c_reshape_and_cache(x[:, 1:2, :].contiguous(), x[:, 1:2, :].contiguous(), kcc, vcc, sl)
    assert same_bits(kc, kcc) and same_bits(vc, vcc)


def test_flash_append_seeded_sweep_of_shapes():
    """Thirty seeded draws of (dtype, block size, heads, head size, tokens, source row stride, fp8 or not, one call per
    layer or one for all): the flash-layout append against the C restatement."""
    g = torch.Generator().manual_seed(4242)
    pick = lambda xs: xs[int(torch.randint(len(xs), (1,), generator=g))]  # noqa: E731
    for case in range(30):
        dtype = pick([torch.bfloat16, torch.float16])
        bs, H, D = pick([1, 4, 16, 32]), pick([1, 2, 3, 4, 8]), pick([3, 8, 40, 64, 80, 128, 256])
        T = pick([1, 2, 17, 64, 255, 256, 257, 1000, 1537, 3000])
        L = pick([1, 2, 5])
        fp8 = pick([False, False, True])
        pad = pick([0, 0, 8, 3])  # extra elements per source row
        fused = pick([True, False])
        NB = T // bs + 9
        say(f"flash append sweep {case}: {dtype} bs={bs} H={H} D={D} T={T} L={L} fp8={fp8} row pad={pad} "
            f"one call for all layers={fused}")
        slots = make_slots(NB * bs, T, 500 + case, pad_frac=0.07)
        src = (torch.randn((L, T, 2 * H * D + pad), generator=g) * 5).to(dtype)
        src_g = src.to(DEV)
        keys = [src_g[l, :, :H * D].view(T, H, D) for l in range(L)]
        values = [src_g[l, :, H * D:2 * H * D].view(T, H, D) for l in range(L)]
        cdt = torch.uint8 if fp8 else dtype
        pool_c = [(torch.arange(2 * NB * bs * H * D) % 53).to(cdt).view(2, NB, bs, H, D).clone() for _ in range(L)]
        pool_g = to_dev(pool_c)
        ks, vs = torch.linspace(0.03, 0.2, L), torch.linspace(0.8, 0.1, L)
        mode = ("fp8", ks, vs) if fp8 else ()
        if fused:
            cache_ops.reshape_and_cache_flash_layers(keys, values, pool_g, slots.to(DEV), *mode)
        else:
            for l in range(L):
                per = ("fp8", ks[l:l + 1].to(DEV), vs[l:l + 1].to(DEV)) if fp8 else ()
                cache_ops.reshape_and_cache_flash(keys[l], values[l], pool_g[l][0], pool_g[l][1], slots.to(DEV), *per)
        for l in range(L):
            k = src[l, :, :H * D].reshape(T, H, D).contiguous()
            v = src[l, :, H * D:2 * H * D].reshape(T, H, D).contiguous()
            if fp8:
                orc.c_reshape_and_cache_fp8(k, v, pool_c[l][0], pool_c[l][1], slots, float(ks[l]), float(vs[l]))
            else:
                orc.c_reshape_and_cache(k, v, pool_c[l][0], pool_c[l][1], slots)
            assert same_bits(pool_g[l], pool_c[l]), f"case {case}, layer {l}"


def test_append_out_of_range_slot_is_skipped():
    kc = torch.full((2, 2, 1, 8), 4.0, dtype=torch.bfloat16, device=DEV)
    vc = kc.clone()
    x = torch.ones((3, 1, 8), dtype=torch.bfloat16, device=DEV)
    cache_ops.reshape_and_cache_flash(x, x, kc, vc, torch.tensor([1, 4, -1], device=DEV))
    want = torch.full((4, 8), 4.0)
    want[1] = 1.0
    assert torch.equal(kc.float().cpu().view(4, 8), want)


# ------------------------------------------------------------------ fp8
def test_append_into_head_major_and_padded_caches():
    """Strided cache views: a head-major pool [NB, H, bs, D] seen as [NB, bs, H, D], and a pool whose
    blocks are padded. The oracle appends into the same views on the CPU; the whole underlying
    storage is compared, so the padding must stay untouched."""
    g = torch.Generator().manual_seed(41)
    # (..., T, L): 500 / 77 tokens: one row per wave; 2000: two, rows of 2 KiB (two passes per row); 6500: four;
    # block size 12 and 40-byte head rows: the division paths (also with two rows per wave: 1700 tokens); 6 heads of
    # 512 bytes: rows of 3 KiB
    for dtype, NB, bs, H, D, T, L in ((torch.bfloat16, 48, 16, 4, 128, 500, 3), (torch.float16, 20, 8, 3, 20, 77, 1),
                                      (torch.bfloat16, 300, 16, 8, 128, 2000, 2), (torch.bfloat16, 500, 16, 4, 128, 6500, 1),
                                      (torch.float16, 30, 12, 2, 64, 100, 2), (torch.float16, 200, 12, 2, 64, 1700, 2),
                                      (torch.bfloat16, 128, 16, 6, 256, 1601, 1)):
        slots = make_slots(NB * bs, T, 41, pad_frac=0.1)
        keys = [torch.randn((T, H, D), generator=g).to(dtype) for _ in range(L)]
        values = [torch.randn((T, H, D), generator=g).to(dtype) for _ in range(L)]
        # head-major storage
        store_c = [torch.full((2, NB, H, bs, D), 3.0, dtype=dtype) for _ in range(L)]
        store_g = [t.to(DEV) for t in store_c]
        for l in range(L):
            kc, vc = store_g[l][0].permute(0, 2, 1, 3), store_g[l][1].permute(0, 2, 1, 3)
            assert not kc.is_contiguous()
            cache_ops.reshape_and_cache_flash(keys[l].to(DEV), values[l].to(DEV), kc, vc, slots.to(DEV), "auto")
            valid = slots >= 0
            b, o = slots[valid] // bs, slots[valid] % bs
            store_c[l][0].permute(0, 2, 1, 3)[b, o] = keys[l][valid]
            store_c[l][1].permute(0, 2, 1, 3)[b, o] = values[l][valid]
            assert same_bits(store_g[l], store_c[l]), f"head-major, layer {l}"
            # brute-force witness on a few tokens
            t = int(valid.nonzero()[0])
            assert torch.equal(store_g[l][0, int(slots[t]) // bs, :, int(slots[t]) % bs, :].cpu(), keys[l][t])
        # padded blocks, all layers in one launch
        pad_c = [torch.full((2, NB, bs + 1, H, D + 8), 5.0, dtype=dtype) for _ in range(L)]
        pad_g = [t.to(DEV) for t in pad_c]
        kv_ops.reshape_and_cache_strided([k.to(DEV) for k in keys], [v.to(DEV) for v in values],
                                         [t[0, :, :bs, :, :D] for t in pad_g], [t[1, :, :bs, :, :D] for t in pad_g],
                                         slots.to(DEV))
        for l in range(L):
            valid = slots >= 0
            b, o = slots[valid] // bs, slots[valid] % bs
            pad_c[l][0, :, :bs, :, :D][b, o] = keys[l][valid]
            pad_c[l][1, :, :bs, :, :D][b, o] = values[l][valid]
            assert same_bits(pad_g[l], pad_c[l]), f"padded, layer {l}"


def test_fp8_append_into_head_major_and_padded_caches():
    """The quantising append into strided fp8 caches: a head-major pool [NB, H, bs, D] seen as [NB, bs, H, D]
    (through the vLLM-shaped call, one layer at a time) and a padded pool (all layers in one launch). Expected
    result = the contiguous fp8 append of the C oracle, permuted: the bytes of a slot's heads are the same, only
    where they lie differs. Both overflow modes, bf16 and f16 sources, head sizes that are not a multiple of 8
    (the element-wise path), block sizes that are not powers of two, rows longer than 1024 elements."""
    g = torch.Generator().manual_seed(43)
    for dtype, NB, bs, H, D, T, L, mode in (
            (torch.bfloat16, 48, 16, 4, 128, 500, 3, "fp8"), (torch.float16, 20, 8, 3, 20, 77, 1, "fp8"),
            (torch.bfloat16, 300, 16, 8, 128, 2000, 2, "fp8_e4m3_sat"), (torch.float16, 30, 12, 2, 64, 100, 2, "fp8_sat"),
            (torch.bfloat16, 64, 16, 6, 256, 601, 1, "fp8"), (torch.bfloat16, 40, 16, 5, 36, 333, 2, "fp8"),
            (torch.float16, 25, 16, 3, 7, 90, 1, "fp8_sat")):
        say(f"fp8 strided append: {dtype} NB={NB} bs={bs} H={H} D={D} T={T} L={L} {mode}")
        sat = mode.endswith("_sat")
        slots = make_slots(NB * bs, T, 43, pad_frac=0.1)
        keys = [(torch.randn((T, H, D), generator=g) * 4).to(dtype) for _ in range(L)]
        values = [(torch.randn((T, H, D), generator=g) * 60).to(dtype) for _ in range(L)]  # part of it overflows
        ks = torch.linspace(0.02, 0.09, L)
        vs = torch.linspace(0.31, 0.11, L)
        # expected: contiguous flash-layout fp8 append of the oracle (the saturating mode through its quantiser)
        flat = [(torch.full((NB, bs, H, D), 9, dtype=torch.uint8), torch.full((NB, bs, H, D), 9, dtype=torch.uint8))
                for _ in range(L)]
        valid = slots >= 0
        b, o = slots[valid] // bs, slots[valid] % bs
        for l in range(L):
            if sat:
                flat[l][0][b, o] = torch.from_numpy(orc.c_quant_fp8_sat(keys[l][valid], float(ks[l]))).view(-1, H, D)
                flat[l][1][b, o] = torch.from_numpy(orc.c_quant_fp8_sat(values[l][valid], float(vs[l]))).view(-1, H, D)
            else:
                orc.c_reshape_and_cache_fp8(keys[l], values[l], flat[l][0], flat[l][1], slots, float(ks[l]), float(vs[l]))
        assert sat or int((flat[0][1] & 0x7F).eq(0x7F).sum()) > 0, "no overflow in the values: the case is too tame"
        # head-major storage, one layer per call
        store_g = [torch.full((2, NB, H, bs, D), 9, dtype=torch.uint8, device=DEV) for _ in range(L)]
        for l in range(L):
            kc = store_g[l][0].permute(0, 2, 1, 3).view(torch.float8_e4m3fn)
            vc = store_g[l][1].permute(0, 2, 1, 3).view(torch.float8_e4m3fn)
            assert not kc.is_contiguous()
            cache_ops.reshape_and_cache_flash(keys[l].to(DEV), values[l].to(DEV), kc, vc, slots.to(DEV), mode,
                                              ks[l:l + 1].to(DEV), vs[l:l + 1].to(DEV))
            assert same_bits(store_g[l][0], flat[l][0].permute(0, 2, 1, 3).contiguous()), f"head-major K, layer {l}"
            assert same_bits(store_g[l][1], flat[l][1].permute(0, 2, 1, 3).contiguous()), f"head-major V, layer {l}"
        # padded blocks, all layers in one launch; the padding must stay untouched
        pad_g = [torch.full((2, NB, bs + 1, H, D + 8), 9, dtype=torch.uint8, device=DEV) for _ in range(L)]
        kv_ops.reshape_and_cache_strided([k.to(DEV) for k in keys], [v.to(DEV) for v in values],
                                         [t[0, :, :bs, :, :D] for t in pad_g], [t[1, :, :bs, :, :D] for t in pad_g],
                                         slots.to(DEV), ks, vs, saturate=sat)
        for l in range(L):
            want = torch.full((2, NB, bs + 1, H, D + 8), 9, dtype=torch.uint8)
            want[0, :, :bs, :, :D] = flat[l][0]
            want[1, :, :bs, :, :D] = flat[l][1]
            assert same_bits(pad_g[l], want), f"padded, layer {l}"
    # a 16-bit cache of another width than the source is still refused
    with pytest.raises(TypeError):
        kv_ops.reshape_and_cache_strided([torch.zeros((1, 1, 8), dtype=torch.float32, device=DEV)] , [torch.zeros((1, 1, 8), dtype=torch.float32, device=DEV)],
                                         [torch.zeros((2, 2, 1, 8), dtype=torch.bfloat16, device=DEV)], [torch.zeros((2, 2, 1, 8), dtype=torch.bfloat16, device=DEV)],
                                         torch.zeros(1, dtype=torch.long, device=DEV))


# ---------------------------------------------------------------- append, paged-attention layout
def paged_slots(NB, bs, T, seed, whole_frac=0.6, pad_frac=0.05, phase=0):
    """A slot table shaped like a serving step: prompts that fill whole blocks in order (the first
    one starts at token `phase`, so block starts are not aligned to token tiles unless phase = 0),
    partial runs, and single scattered tokens; a few padded entries."""
    g = torch.Generator().manual_seed(seed)
    blocks = torch.randperm(NB, generator=g).tolist()
    slots = []
    for _ in range(phase):
        b = blocks.pop()
        slots.append(b * bs + int(torch.randint(bs, (1,), generator=g)))
    while len(slots) < T * whole_frac and blocks:
        b = blocks.pop()
        slots.extend(range(b * bs, (b + 1) * bs))
    while len(slots) < T and blocks:
        b = blocks.pop()
        run = int(torch.randint(1, bs + 1, (1,), generator=g))
        start = int(torch.randint(0, bs - run + 1, (1,), generator=g))
        slots.extend(range(b * bs + start, b * bs + start + run))
    slots = torch.tensor(slots[:T], dtype=torch.long)
    pad = torch.rand(len(slots), generator=g) < pad_frac
    slots[pad] = -1
    return slots


def paged_caches_cpu(NB, H, D, bs, dtype, fill_mod=61):
    eb = 1 if dtype == torch.uint8 else 2
    x = 16 // eb
    n = NB * H * D * bs
    base = (torch.arange(n, dtype=torch.float32) % fill_mod)
    base = base.to(torch.uint8) if dtype == torch.uint8 else base.to(dtype)
    return base.view(NB, H, D // x, bs, x).clone(), base.view(NB, H, D, bs).clone()


@pytest.mark.parametrize("dtype,NB,bs,H,D,T,phase,desc", [
    (torch.bfloat16, 1024, 16, 4, 128, 8448, 0, "Qwen2-7B rows, prompts aligned to token tiles"),
    (torch.bfloat16, 1024, 16, 4, 128, 8448, 5, "Qwen2-7B rows, prompts off the tile grid"),
    (torch.float16, 300, 16, 8, 128, 2500, 3, "70B-shape rows: two row segments per token"),
    (torch.float16, 96, 8, 3, 40, 333, 0, "120-element rows, block size 8"),
    (torch.bfloat16, 48, 32, 2, 64, 700, 0, "block size 32"),
    (torch.bfloat16, 33, 16, 5, 104, 1, 0, "a single token; 520-element rows (second segment of 8)"),
    (torch.bfloat16, 64, 16, 4, 128, 256, 5, "256 tokens (tiles of 4 tokens): prompts off the tile grid"),
    (torch.float16, 64, 16, 8, 128, 200, 0, "200 tokens (tiles of 4 tokens), two row segments"),
    (torch.float16, 96, 8, 3, 40, 150, 3, "150 tokens (tiles of 4 tokens), block size 8"),
    (torch.bfloat16, 48, 32, 2, 64, 250, 1, "250 tokens (tiles of 4 tokens), block size 32"),
])
def test_paged_append_against_oracle(dtype, NB, bs, H, D, T, phase, desc):
    say(f"paged append: {desc}")
    g = torch.Generator().manual_seed(NB + T)
    key = torch.randn((T, H, D), generator=g).to(dtype)
    value = torch.randn((T, H, D), generator=g).to(dtype)
    slots = paged_slots(NB, bs, T, seed=T, phase=phase)
    assert len(slots) == T
    kc, vc = paged_caches_cpu(NB, H, D, bs, dtype)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    cache_ops.reshape_and_cache(key.to(DEV), value.to(DEV), kc_g, vc_g, slots.to(DEV), "auto")
    orc.c_reshape_and_cache_paged(key, value, kc, vc, slots)
    assert same_bits(kc_g, kc) and same_bits(vc_g, vc)
    if T <= 2500:  # the torch statement as a second witness
        kr, vr = paged_caches_cpu(NB, H, D, bs, dtype)
        orc.ref_reshape_and_cache_paged(key, value, kr, vr, slots)
        assert same_bits(kc_g, kr) and same_bits(vc_g, vr)


def test_paged_append_strided_sources_random_slots_and_golden(golden_dir):
    NB, bs, H, D, T = 24, 16, 2, 64, 101
    g = torch.Generator().manual_seed(77)
    qkv = torch.randn((T, 3 * H * D + 4), generator=g).to(torch.float16)  # row stride not a multiple of 8 elements
    slots = make_slots(NB * bs, T, 77, pad_frac=0.1)
    qkv_g = qkv.to(DEV)
    for lo in (H * D, H * D + 1):  # second view: base not 16-byte aligned
        k_g = qkv_g[:, lo:lo + H * D].view(T, H, D)
        v_g = qkv_g[:, lo + H * D:lo + 2 * H * D].view(T, H, D)
        kc, vc = paged_caches_cpu(NB, H, D, bs, torch.float16)
        kc_g, vc_g = kc.to(DEV), vc.to(DEV)
        cache_ops.reshape_and_cache(k_g, v_g, kc_g, vc_g, slots.to(DEV))
        orc.c_reshape_and_cache_paged(qkv[:, lo:lo + H * D].reshape(T, H, D).contiguous(),
                                      qkv[:, lo + H * D:lo + 2 * H * D].reshape(T, H, D).contiguous(), kc, vc, slots)
        assert same_bits(kc_g, kc) and same_bits(vc_g, vc)
    z = np.load(os.path.join(golden_dir, "paged_small.npz"))
    bf = torch.bfloat16
    as_t = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(bf)  # noqa: E731
    kc_g, vc_g = as_t(z["key_cache_before"]).to(DEV), as_t(z["value_cache_before"]).to(DEV)
    cache_ops.reshape_and_cache(as_t(z["key"]).to(DEV), as_t(z["value"]).to(DEV), kc_g, vc_g,
                                torch.from_numpy(z["slots"]).to(DEV))
    assert same_bits(kc_g, z["key_cache_after"]) and same_bits(vc_g, z["value_cache_after"])
    # a slot past the pool and an empty call
    kc_g2 = kc_g.clone()
    x = torch.ones((2, kc_g.shape[1], kc_g.shape[2] * kc_g.shape[4]), dtype=bf, device=DEV)
    cache_ops.reshape_and_cache(x, x, kc_g2, vc_g, torch.tensor([kc_g.shape[0] * kc_g.shape[3], -1], device=DEV))
    cache_ops.reshape_and_cache(x[:0], x[:0], kc_g2, vc_g, torch.empty(0, dtype=torch.long, device=DEV))
    assert torch.equal(kc_g2, kc_g)


@pytest.mark.parametrize("T,fp8", [(700, False), (200, False), (700, True), (200, True)])
def test_paged_append_unaligned_sources_with_whole_runs(T, fp8):
    """Sources that do not allow 16-byte loads (odd row stride, base off by one element) with prompts that
    fill blocks: the element-wise source path feeds both the staged whole runs and the direct stores, with
    tiles of 16 (700 tokens) and of 4 tokens (200)."""
    NB, bs, H, D = 64, 16, 2, 128
    g = torch.Generator().manual_seed(T)
    qkv = (torch.randn((T, 2 * H * D + 3), generator=g) * 3).to(torch.bfloat16)
    slots = paged_slots(NB, bs, T, seed=T + 1, phase=3)
    key, value = qkv[:, 1:1 + H * D], qkv[:, 1 + H * D:1 + 2 * H * D]
    cdt = torch.uint8 if fp8 else torch.bfloat16
    kc, vc = paged_caches_cpu(NB, H, D, bs, cdt)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    qkv_g = qkv.to(DEV)
    k_g, v_g = qkv_g[:, 1:1 + H * D].view(T, H, D), qkv_g[:, 1 + H * D:1 + 2 * H * D].view(T, H, D)
    ks, vs = torch.tensor([0.07]), torch.tensor([0.3])
    if fp8:
        cache_ops.reshape_and_cache(k_g, v_g, kc_g.view(torch.float8_e4m3fn), vc_g.view(torch.float8_e4m3fn),
                                    slots.to(DEV), "fp8", ks.to(DEV), vs.to(DEV))
        orc.c_reshape_and_cache_paged(key.reshape(T, H, D).contiguous(), value.reshape(T, H, D).contiguous(), kc, vc,
                                      slots, float(ks), float(vs))
    else:
        cache_ops.reshape_and_cache(k_g, v_g, kc_g, vc_g, slots.to(DEV))
        orc.c_reshape_and_cache_paged(key.reshape(T, H, D).contiguous(), value.reshape(T, H, D).contiguous(), kc, vc,
                                      slots)
    assert same_bits(kc_g, kc) and same_bits(vc_g, vc)


@pytest.mark.parametrize("bs,T,first", [(16, 2048, 0), (16, 2048, 11), (8, 900, 3), (32, 1500, 17), (16, 250, 9)])
def test_paged_append_slots_in_pool_order(bs, T, first):
    """A fresh block manager hands out blocks 0, 1, 2, ...: the slots of a prompt are then consecutive across
    block boundaries, and a run of consecutive slots must still end at every block's end. Also the same
    slots backwards (consecutive downwards: no runs at all), and every other slot."""
    NB, H, D = 160, 4, 128
    g = torch.Generator().manual_seed(bs + T)
    key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    up = torch.arange(first, first + T, dtype=torch.long)
    for name, slots in (("ascending", up), ("descending", up.flip(0).contiguous()),
                        ("every other slot", (up * 2) % (NB * bs - 1))):
        say(f"paged append, slots in pool order: block size {bs}, {T} tokens from slot {first}, {name}")
        if name == "every other slot":
            slots = torch.unique(slots, sorted=False)[:T]  # no slot twice: the order of two writes is not defined
        n = len(slots)
        kc, vc = paged_caches_cpu(NB, H, D, bs, torch.bfloat16)
        kc_g, vc_g = kc.to(DEV), vc.to(DEV)
        cache_ops.reshape_and_cache(key[:n].to(DEV), value[:n].to(DEV), kc_g, vc_g, slots.to(DEV))
        orc.c_reshape_and_cache_paged(key[:n].contiguous(), value[:n].contiguous(), kc, vc, slots)
        assert same_bits(kc_g, kc) and same_bits(vc_g, vc), name


@pytest.mark.parametrize("bs", [1, 4, 24, 40, 64, 128])
@pytest.mark.parametrize("fp8", [False, True])
def test_paged_append_unusual_block_sizes(bs, fp8):
    """Block sizes outside 8 / 16 / 32, not all powers of two: runs still end at every block's end and at every
    16th slot of a block, and a 16-token run is staged as a whole only where its V region is 16-byte aligned."""
    NB, H, D, T = 2200 // bs + 30, 2, 128, 900
    g = torch.Generator().manual_seed(bs)
    key = (torch.randn((T, H, D), generator=g) * 2).to(torch.bfloat16)
    value = (torch.randn((T, H, D), generator=g) * 2).to(torch.bfloat16)
    slots = paged_slots(NB, bs, T, seed=bs, phase=2)
    assert len(slots) == T
    kc, vc = paged_caches_cpu(NB, H, D, bs, torch.uint8 if fp8 else torch.bfloat16)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    if fp8:
        ks, vs = torch.tensor([0.05]), torch.tensor([0.2])
        cache_ops.reshape_and_cache(key.to(DEV), value.to(DEV), kc_g.view(torch.float8_e4m3fn),
                                    vc_g.view(torch.float8_e4m3fn), slots.to(DEV), "fp8", ks.to(DEV), vs.to(DEV))
        orc.c_reshape_and_cache_paged(key, value, kc, vc, slots, float(ks), float(vs))
    else:
        cache_ops.reshape_and_cache(key.to(DEV), value.to(DEV), kc_g, vc_g, slots.to(DEV))
        orc.c_reshape_and_cache_paged(key, value, kc, vc, slots)
    assert same_bits(kc_g, kc) and same_bits(vc_g, vc)


@pytest.mark.parametrize("width", [1, 2], ids=["256 row elements per workgroup", "128 row elements per workgroup"])
def test_paged_append_both_tile_widths(width, monkeypatch):
    """A one-layer launch takes workgroups of 128 row elements while it fits the device at once and of 256 beyond;
    here each width is forced (test hook of the hooks library) on launches of either size, tiles of 4 and of 16
    tokens, 16-bit and fp8 caches, rows that end inside a workgroup's segment, misaligned sources."""
    hooks = _lib.load_hooks()
    monkeypatch.setattr(_lib, "_lib", hooks)
    old = hooks.emm_hook_set_move_variant((width << 22) | (1 << 28))  # bit 28: the general kernel for every shape
    try:
        for (dtype, NB, bs, H, D, T, phase, fp8, pad) in [
                (torch.bfloat16, 700, 16, 4, 128, 5000, 3, False, 0), (torch.float16, 300, 16, 8, 128, 2500, 0, True, 0),
                (torch.bfloat16, 200, 16, 4, 128, 1000, 7, False, 0), (torch.bfloat16, 64, 16, 4, 128, 256, 5, False, 0),
                (torch.float16, 96, 8, 3, 40, 333, 0, False, 0), (torch.bfloat16, 33, 16, 5, 112, 77, 2, True, 0), (torch.bfloat16, 33, 16, 5, 104, 77, 2, False, 0),
                (torch.bfloat16, 48, 32, 2, 64, 700, 1, False, 8), (torch.float16, 80, 16, 3, 96, 300, 4, False, 5),
                (torch.bfloat16, 40, 16, 1, 64, 130, 0, True, 5), (torch.bfloat16, 30, 16, 20, 128, 100, 1, False, 0)]:
            say(f"paged append, width code {width}: {dtype} NB={NB} bs={bs} H={H} D={D} T={T} fp8={fp8} row pad={pad}")
            g = torch.Generator().manual_seed(NB * 7 + T + width)
            slots = paged_slots(NB, bs, T, seed=T + 1, phase=phase)
            src = (torch.randn((T, 2 * H * D + pad), generator=g) * 3).to(dtype)
            src_g = src.to(DEV)
            k_g, v_g = src_g[:, :H * D].view(T, H, D), src_g[:, H * D:2 * H * D].view(T, H, D)
            kh = src[:, :H * D].reshape(T, H, D).contiguous()
            vh = src[:, H * D:2 * H * D].reshape(T, H, D).contiguous()
            kc, vc = paged_caches_cpu(NB, H, D, bs, torch.uint8 if fp8 else dtype)
            kc_g, vc_g = kc.to(DEV), vc.to(DEV)
            if fp8:
                ks, vs = torch.tensor([0.07]), torch.tensor([0.6])
                cache_ops.reshape_and_cache(k_g, v_g, kc_g.view(torch.float8_e4m3fn), vc_g.view(torch.float8_e4m3fn),
                                            slots.to(DEV), "fp8", ks.to(DEV), vs.to(DEV))
                orc.c_reshape_and_cache_paged(kh, vh, kc, vc, slots, float(ks), float(vs))
            else:
                cache_ops.reshape_and_cache(k_g, v_g, kc_g, vc_g, slots.to(DEV))
                orc.c_reshape_and_cache_paged(kh, vh, kc, vc, slots)
            assert same_bits(kc_g, kc) and same_bits(vc_g, vc), f"T={T} H={H} D={D} fp8={fp8}"
    finally:
        hooks.emm_hook_set_move_variant(old)


@pytest.mark.parametrize("cols,fused", [(1, 1), (1, 2), (2, 1), (2, 2), (3, 1), (3, 2)],
                         ids=["128 row elements, K and V in one wave", "128 row elements, K and V in two waves",
                              "32 row elements, one wave", "32 row elements, two waves",
                              "256 row elements, one wave", "256 row elements, two waves"])
def test_paged_append_one_wave_kernel_every_wave_shape(cols, fused, monkeypatch):
    """16-bit caches with aligned sources and a power-of-two block size from 16 on take the kernel of one-wave
    workgroups, which picks how many row elements a wave takes, and whether K and V share a wave, by launch size;
    here each shape is forced on launches of either size: rows that end inside a column, strided sources, prompts
    on and off the token-tile grid, block size 32 and 64."""
    hooks = _lib.load_hooks()
    monkeypatch.setattr(_lib, "_lib", hooks)
    old = hooks.emm_hook_set_move_variant((cols << 29) | (fused << 20))
    try:
        for (dtype, NB, bs, H, D, T, phase, pad) in [
                (torch.bfloat16, 700, 16, 4, 128, 5000, 3, 0), (torch.float16, 300, 16, 8, 128, 2500, 0, 0),
                (torch.bfloat16, 64, 16, 4, 128, 256, 5, 0), (torch.bfloat16, 33, 16, 5, 104, 77, 2, 0),
                (torch.float16, 80, 16, 3, 40, 300, 4, 8), (torch.bfloat16, 48, 32, 2, 64, 700, 1, 8),
                (torch.bfloat16, 60, 64, 1, 72, 900, 15, 0), (torch.bfloat16, 30, 16, 20, 128, 100, 1, 0),
                (torch.float16, 40, 16, 1, 8, 333, 0, 0)]:
            say(f"paged append, one-wave kernel, column code {cols}, fused code {fused}: {dtype} NB={NB} bs={bs} H={H} D={D} "
                f"T={T} pad={pad}")
            g = torch.Generator().manual_seed(NB * 7 + T + cols)
            slots = paged_slots(NB, bs, T, seed=T + 1, phase=phase)
            assert len(slots) == T
            src = (torch.randn((T, 2 * H * D + pad), generator=g) * 3).to(dtype)
            src_g = src.to(DEV)
            k_g, v_g = src_g[:, :H * D].view(T, H, D), src_g[:, H * D:2 * H * D].view(T, H, D)
            kh = src[:, :H * D].reshape(T, H, D).contiguous()
            vh = src[:, H * D:2 * H * D].reshape(T, H, D).contiguous()
            kc, vc = paged_caches_cpu(NB, H, D, bs, dtype)
            kc_g, vc_g = kc.to(DEV), vc.to(DEV)
            cache_ops.reshape_and_cache(k_g, v_g, kc_g, vc_g, slots.to(DEV))
            orc.c_reshape_and_cache_paged(kh, vh, kc, vc, slots)
            assert same_bits(kc_g, kc) and same_bits(vc_g, vc), f"T={T} H={H} D={D}"
    finally:
        hooks.emm_hook_set_move_variant(old)


def test_paged_append_runs_at_every_position_and_broken_runs():
    """What decides between the whole-run path and token-by-token stores, one case at a time: a 16-token run
    starting at every position of the token list relative to the 16-token tiles, at the very start and the very
    end of the list, runs that only look whole (a padded slot, a repeated slot, a slot past the pool, a gap, a
    start that is not a multiple of 16 slots inside a block of 32), two whole runs back to back, and 17 / 31 / 32
    consecutive slots."""
    NB, bs, H, D = 40, 32, 2, 64
    g = torch.Generator().manual_seed(1234)
    cases = []
    for start in range(0, 34):  # `start` single tokens, then one whole run, then 3 single tokens
        lone = [(3 + i) * bs + 20 for i in range(start)]  # never inside the run's window
        cases.append((f"run at token {start}", lone + list(range(20 * bs, 20 * bs + 16)) + [30 * bs + 1, 31 * bs + 2, 32 * bs + 3]))
    run = list(range(20 * bs + 16, 20 * bs + 32))  # the second 16-slot window of block 20
    cases.append(("run alone", run))
    cases.append(("run at the end", [5, 70, 200] + run))
    broken = list(run); broken[9] = -1
    cases.append(("padded slot inside", [1] * 0 + broken + [99]))
    broken = list(run); broken[4] = broken[3]
    cases.append(("repeated slot inside", broken[:4] + broken[5:]))  # 15 tokens, consecutive except one step of 2
    broken = list(run); broken[15] = NB * bs + 5
    cases.append(("last slot past the pool", broken))
    cases.append(("gap in the middle", run[:8] + [700] + run[8:]))
    cases.append(("start not at a window start", list(range(20 * bs + 8, 20 * bs + 24))))
    cases.append(("two runs back to back", list(range(20 * bs, 20 * bs + 32))))
    cases.append(("two runs, other order", list(range(20 * bs + 16, 20 * bs + 32)) + list(range(20 * bs, 20 * bs + 16))))
    for n in (15, 17, 31, 32, 33, 47, 48, 49, 64):
        cases.append((f"{n} consecutive slots from 5", list(range(9 * bs + 5, 9 * bs + 5 + n))))
        cases.append((f"{n} consecutive slots from a block start", list(range(9 * bs, 9 * bs + n))))
    for name, sl in cases:
        say(f"paged append, run edges: {name}")
        slots = torch.tensor(sl, dtype=torch.long)
        T = len(sl)
        key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
        value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
        kc, vc = paged_caches_cpu(NB, H, D, bs, torch.bfloat16)
        kc_g, vc_g = kc.to(DEV), vc.to(DEV)
        cache_ops.reshape_and_cache(key.to(DEV), value.to(DEV), kc_g, vc_g, slots.to(DEV))
        orc.c_reshape_and_cache_paged(key, value, kc, vc, slots)
        assert same_bits(kc_g, kc) and same_bits(vc_g, vc), name


def test_paged_append_seeded_sweep_of_shapes():
    """Forty seeded draws of (dtype, block size, heads, head size, tokens, slot pattern, fp8 or not, source
    row stride), each against the C restatement: shapes nobody picked by hand."""
    g = torch.Generator().manual_seed(20240607)
    pick = lambda xs: xs[int(torch.randint(len(xs), (1,), generator=g))]  # noqa: E731
    for case in range(40):
        dtype = pick([torch.bfloat16, torch.float16])
        bs = pick([8, 16, 16, 16, 32])
        H = pick([1, 2, 3, 4, 8])
        D = pick([32, 64, 80, 96, 128, 256])
        T = pick([1, 2, 15, 16, 17, 63, 255, 256, 257, 600, 1100])
        fp8 = pick([False, False, True])
        pad = pick([0, 0, 8, 5])  # extra elements per source row: 5 forbids 16-byte loads
        phase = pick([0, 1, 7, 15])
        whole = pick([0.0, 0.5, 1.0])
        NB = 3 * T // bs + 60
        say(f"paged sweep {case}: {dtype} bs={bs} H={H} D={D} T={T} fp8={fp8} row pad={pad} phase={phase} "
            f"whole={whole}")
        slots = paged_slots(NB, bs, T, seed=1000 + case, whole_frac=whole, phase=min(phase, T))
        src = (torch.randn((T, 2 * H * D + pad), generator=g) * 3).to(dtype)
        key, value = src[:, :H * D], src[:, H * D:2 * H * D]
        src_g = src.to(DEV)
        k_g, v_g = src_g[:, :H * D].view(T, H, D), src_g[:, H * D:2 * H * D].view(T, H, D)
        cdt = torch.uint8 if fp8 else dtype
        kc, vc = paged_caches_cpu(NB, H, D, bs, cdt)
        kc_g, vc_g = kc.to(DEV), vc.to(DEV)
        kh, vh = key.reshape(T, H, D).contiguous(), value.reshape(T, H, D).contiguous()
        if fp8:
            ks, vs = torch.tensor([0.04 + 0.01 * case]), torch.tensor([0.9 - 0.02 * case])
            cache_ops.reshape_and_cache(k_g, v_g, kc_g.view(torch.float8_e4m3fn), vc_g.view(torch.float8_e4m3fn),
                                        slots.to(DEV), "fp8", ks.to(DEV), vs.to(DEV))
            orc.c_reshape_and_cache_paged(kh, vh, kc, vc, slots, float(ks), float(vs))
        else:
            cache_ops.reshape_and_cache(k_g, v_g, kc_g, vc_g, slots.to(DEV))
            orc.c_reshape_and_cache_paged(kh, vh, kc, vc, slots)
        assert same_bits(kc_g, kc) and same_bits(vc_g, vc), f"case {case}"


@pytest.mark.parametrize("fp8", [False, True])
def test_paged_append_all_layers_in_one_launch(fp8):
    L, NB, bs, H, D, T = 5, 96, 16, 2, 128, 900
    g = torch.Generator().manual_seed(31)
    slots = paged_slots(NB, bs, T, seed=31, phase=7)
    keys = [(torch.randn((T, H, D), generator=g) * 2).to(torch.bfloat16) for _ in range(L)]
    values = [(torch.randn((T, H, D), generator=g) * 2).to(torch.bfloat16) for _ in range(L)]
    ks = torch.linspace(0.02, 0.08, L)
    vs = torch.linspace(0.5, 0.1, L)
    cdt = torch.uint8 if fp8 else torch.bfloat16
    caches = [paged_caches_cpu(NB, H, D, bs, cdt, fill_mod=31 + l) for l in range(L)]
    kcs = [c[0].to(DEV) for c in caches]
    vcs = [c[1].to(DEV) for c in caches]
    plan = cache_ops.paged_layered_append([k.to(DEV) for k in keys], [v.to(DEV) for v in values], kcs, vcs,
                                          "fp8" if fp8 else "auto", ks, vs)
    plan(slots.to(DEV))
    for l in range(L):
        kc, vc = caches[l]
        orc.c_reshape_and_cache_paged(keys[l], values[l], kc, vc, slots, float(ks[l]), float(vs[l]))
        assert same_bits(kcs[l], kc) and same_bits(vcs[l], vc), f"layer {l}"


@pytest.mark.parametrize("dtype,phase,T", [(torch.bfloat16, 0, 2000), (torch.float16, 2, 2000),
                                           (torch.bfloat16, 3, 256), (torch.float16, 0, 77)])
def test_paged_append_fp8(dtype, phase, T):
    NB, bs, H, D = 200, 16, 4, 128
    g = torch.Generator().manual_seed(5)
    key = (torch.randn((T, H, D), generator=g) * 4).to(dtype)
    value = (torch.randn((T, H, D), generator=g) * 300).to(dtype)  # part of it overflows to NaN
    slots = paged_slots(NB, bs, T, seed=9, phase=phase, pad_frac=0.01)
    ks, vs = torch.tensor([0.05]), torch.tensor([0.61])
    kc, vc = paged_caches_cpu(NB, H, D, bs, torch.uint8)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    cache_ops.reshape_and_cache(key.to(DEV), value.to(DEV), kc_g.view(torch.float8_e4m3fn),
                                vc_g.view(torch.float8_e4m3fn), slots.to(DEV), "fp8", ks.to(DEV), vs.to(DEV))
    orc.c_reshape_and_cache_paged(key, value, kc, vc, slots, float(ks), float(vs))
    assert same_bits(kc_g, kc) and same_bits(vc_g, vc)
    kr, vr = paged_caches_cpu(NB, H, D, bs, torch.uint8)
    orc.ref_reshape_and_cache_paged(key, value, kr, vr, slots, "fp8", ks, vs)
    assert same_bits(kc_g, kr) and same_bits(vc_g, vr)
    assert int((vc_g.cpu() & 0x7F).eq(0x7F).sum()) > (100 if T >= 2000 else 3)


def test_fp8_append_exhaustive_bf16_and_f16(golden_dir):
    """Every 16-bit input x several scales through the append kernel: 64 tokens x 1024
    elements is exactly the 65 536 bit patterns."""
    kat = json.load(open(os.path.join(golden_dir, "fp8_kat.json")))
    import hashlib
    for dtype, name in ((torch.bfloat16, "bf16"), (torch.float16, "f16")):
        allx = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
        key = allx.view(64, 8, 128)
        value = allx.flip(0).contiguous().view(64, 8, 128)
        slots = torch.arange(64)
        for s in kat["scales"]:
            say(f"fp8 exhaustive {name} scale {s}")
            kc = torch.zeros((4, 16, 8, 128), dtype=torch.uint8, device=DEV)
            vc = torch.zeros_like(kc)
            sc = torch.tensor([s], dtype=torch.float32, device=DEV)
            cache_ops.reshape_and_cache_flash(key.to(DEV), value.to(DEV), kc.view(torch.float8_e4m3fn),
                                              vc.view(torch.float8_e4m3fn), slots.to(DEV), "fp8", sc, sc)
            got = raw(kc)
            want = orc.c_quant_fp8(allx, s).reshape(-1)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, f"{name} scale {s}: {bad.size} mismatches, first bits {bad[:8]} got {got[bad[:8]]} want {want[bad[:8]]}"
            assert hashlib.sha256(got.tobytes()).hexdigest() == kat["sweep_sha256"][f"{name}@{s}"]
            assert (raw(vc) == orc.c_quant_fp8(allx.flip(0).contiguous(), s).reshape(-1)).all()


def test_fp8_known_answers_on_gpu():
    xs = [448, 464, 465, 480, -1000, 2 ** -9, 2 ** -10, 2 ** -10 * 1.0001, 17, 18, 19, float("inf")]
    want = [126, 126, 127, 127, 255, 1, 0, 1, 88, 89, 90, 127]
    x = torch.zeros((1, 1, 16), dtype=torch.bfloat16)
    x[0, 0, :12] = torch.tensor(xs, dtype=torch.float32).to(torch.bfloat16)
    # 465 and 2^-10*1.0001 are not bf16 values: use f32-exact neighbours that are
    x[0, 0, 2] = 466.0
    x[0, 0, 7] = 2 ** -10 * 1.0078125
    kc = torch.zeros((1, 1, 1, 16), dtype=torch.uint8, device=DEV)
    vc = torch.zeros_like(kc)
    one = torch.ones(1, device=DEV)
    cache_ops.reshape_and_cache_flash(x.to(DEV), x.to(DEV), kc, vc, torch.zeros(1, dtype=torch.long, device=DEV),
                                      "fp8", one, one)
    assert raw(kc)[:12].tolist() == want


def test_cfg4_fp8_append_pack_dequant_reduced():
    say("cfg4 shape reduced: 6 layers [2,256,16,8,128] fp8, scales U[0.01,0.1], T=1500")
    L, NB, bs, H, D, T = 6, 256, 16, 8, 128, 1500
    g = torch.Generator().manual_seed(4)
    ks = (torch.rand(L, generator=g) * 0.09 + 0.01).float()
    vs = (torch.rand(L, generator=g) * 0.09 + 0.01).float()
    slots = make_slots(NB * bs, T, 4)
    pool_c = [torch.full((2, NB, bs, H, D), 0x5A, dtype=torch.uint8) for _ in range(L)]
    pool_g = to_dev(pool_c)
    keys, values = [], []
    for l in range(L):
        k = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
        v = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
        keys.append(k.to(DEV))
        values.append(v.to(DEV))
        orc.c_reshape_and_cache_fp8(k, v, pool_c[l][0], pool_c[l][1], slots, float(ks[l]), float(vs[l]))
    # layer 0 through the per-layer entry point, all through the fused one on a second pool
    pool_g2 = [p.clone() for p in pool_g]
    for l in range(L):
        cache_ops.reshape_and_cache_flash(keys[l], values[l], pool_g[l][0], pool_g[l][1], slots.to(DEV), "fp8",
                                          ks[l:l + 1].to(DEV), vs[l:l + 1].to(DEV))
    cache_ops.reshape_and_cache_flash_layers(keys, values, pool_g2, slots.to(DEV), "fp8", ks, vs)
    for l in range(L):
        assert same_bits(pool_g[l], pool_c[l]), f"layer {l}"
        assert same_bits(pool_g2[l], pool_c[l]), f"fused layer {l}"
    # pack / unpack move fp8 bytes
    si = torch.randperm(NB, generator=g)[:40].tolist()
    di = torch.randperm(NB, generator=g)[:40].tolist()
    packed = kv_ops.kv_pack(PoolView(pool_g), si)
    assert packed.dtype == torch.uint8 and same_bits(packed, orc.c_kv_pack(pool_c, si))
    dst8 = [torch.zeros_like(p) for p in pool_g]
    kv_ops.kv_unpack(PoolView(dst8), di, packed)
    dst8_c = [torch.zeros_like(p) for p in pool_c]
    orc.c_kv_unpack(dst8_c, di, raw(packed))
    assert same_bits(torch.stack(dst8), torch.stack(dst8_c))
    # dequantising unpack into bf16 and f16 pools
    for dt in (torch.bfloat16, torch.float16):
        dq_g = [torch.full((2, NB, bs, H, D), 9.0, dtype=dt, device=DEV) for _ in range(L)]
        dq_c = [torch.full((2, NB, bs, H, D), 9.0, dtype=dt) for _ in range(L)]
        kv_ops.kv_unpack_dequant_fp8(PoolView(dq_g), di, packed, ks, vs)
        orc.c_unpack_dequant_fp8(dq_c, di, raw(packed), ks.numpy(), vs.numpy())
        assert same_bits(torch.stack(dq_g), torch.stack(dq_c)), str(dt)


@pytest.mark.parametrize("bit,name", [(0x1000, "whole-row waves"), (0x2000, "512-element waves")])
def test_fp8_append_both_wave_shapes(bit, name, monkeypatch):
    """The fp8 append picks between waves that convert a whole row (pieces of 1024 elements) and waves that convert
    512 elements by launch size; here each is forced, per layer and as one launch for all layers, on rows that end
    inside a piece, rows longer than two pieces, strided sources, padded slots and both overflow modes."""
    hooks = _lib.load_hooks()
    monkeypatch.setattr(_lib, "_lib", hooks)
    old = hooks.emm_hook_set_move_variant(bit)
    try:
        for (dtype, L, NB, bs, H, D, T, pad, mode) in [
                (torch.bfloat16, 3, 64, 16, 8, 128, 700, 0, "fp8"), (torch.float16, 2, 40, 16, 5, 104, 333, 8, "fp8"),
                (torch.bfloat16, 2, 20, 16, 1, 8, 100, 0, "fp8_e4m3_sat"), (torch.bfloat16, 2, 24, 8, 20, 128, 150, 0, "fp8"),
                (torch.float16, 1, 16, 16, 3, 200, 77, 16, "fp8_e4m3_sat"), (torch.bfloat16, 2, 200, 16, 8, 128, 2500, 0, "fp8")]:
            say(f"fp8 append, {name}: {dtype} L={L} NB={NB} bs={bs} H={H} D={D} T={T} pad={pad} {mode}")
            g = torch.Generator().manual_seed(NB + T)
            ks = (torch.rand(L, generator=g) * 0.09 + 0.01).float()
            vs = (torch.rand(L, generator=g) * 0.09 + 0.01).float()
            slots = make_slots(NB * bs, T, T)
            pool_c = [torch.full((2, NB, bs, H, D), 0x5A, dtype=torch.uint8) for _ in range(L)]
            pool_g, pool_g2 = to_dev(pool_c), to_dev(pool_c)
            keys, values = [], []
            for l in range(L):
                src = (torch.randn((T, 2 * H * D + pad), generator=g) * 40).to(dtype)
                src[::17, ::5] = 1e30 if dtype == torch.bfloat16 else 60000.0  # overflows of both signs
                src[3::19, 1::7] *= -1
                src_g = src.to(DEV)
                keys.append(src_g[:, :H * D].view(T, H, D))
                values.append(src_g[:, H * D:2 * H * D].view(T, H, D))
                quant = orc.c_quant_fp8_sat if mode.endswith("sat") else orc.c_quant_fp8
                live = slots >= 0  # the slots are distinct: a plain scatter of the quantised rows is the append
                for kv, lo, scale in ((0, 0, ks[l]), (1, H * D, vs[l])):
                    q = torch.from_numpy(quant(src[:, lo:lo + H * D].contiguous(), float(scale)))
                    pool_c[l][kv].view(NB * bs, H * D)[slots[live]] = q[live]
                cache_ops.reshape_and_cache_flash(keys[l], values[l], pool_g[l][0], pool_g[l][1], slots.to(DEV), mode,
                                                  ks[l:l + 1].to(DEV), vs[l:l + 1].to(DEV))
            cache_ops.reshape_and_cache_flash_layers(keys, values, pool_g2, slots.to(DEV), mode, ks, vs)
            for l in range(L):
                assert same_bits(pool_g[l], pool_c[l]), f"per layer, layer {l}"
                assert same_bits(pool_g2[l], pool_c[l]), f"one launch, layer {l}"
    finally:
        hooks.emm_hook_set_move_variant(old)


def test_fp8_dequant_all_bytes_all_scales(golden_dir):
    kat = json.load(open(os.path.join(golden_dir, "fp8_kat.json")))
    scales = kat["scales"]
    L = len(scales)
    # one block of 256 bytes per layer holding every byte value; K uses scale s, V uses s/3
    allq = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    packed = allq.view(1, 1, 1, 256).expand(L, 2, 1, 256).contiguous().to(DEV)
    ks = torch.tensor(scales, dtype=torch.float32)
    vs = ks / 3
    for dt in (torch.bfloat16, torch.float16):
        pool = [torch.zeros((2, 2, 1, 2, 128), dtype=dt, device=DEV) for _ in range(L)]
        kv_ops.kv_unpack_dequant_fp8(PoolView(pool), [1], packed, ks, vs)
        for l, s in enumerate(scales):
            got = pool[l].cpu().view(torch.int16).numpy().view(np.uint16)
            assert (got[0, 1].reshape(-1) == orc.c_dequant_fp8(allq.numpy(), float(ks[l]), dt)).all()
            assert (got[1, 1].reshape(-1) == orc.c_dequant_fp8(allq.numpy(), float(vs[l]), dt)).all()
            assert not got[:, 0].any()
            if dt == torch.bfloat16 and f"bf16@{s}" in kat["dequant"]:
                assert got[0, 1].reshape(-1).tolist() == kat["dequant"][f"bf16@{s}"]


# ------------------------------------------------------------------ vision concat
def test_concat_rows_ragged():
    say("vision concat: 20 tensors [U{64..2304}, 3584] bf16 + edge cases")
    g = torch.Generator().manual_seed(5)
    rows = torch.randint(64, 2305, (20,), generator=g).tolist()
    segs = [torch.randn((r, 3584), generator=g).to(torch.bfloat16) for r in rows]
    got = kv_ops.concat_rows([s.to(DEV) for s in segs])
    assert got.shape == (sum(rows), 3584)
    assert same_bits(got, orc.ref_concat_rows(segs))
    # more segments than one launch carries, with empty and odd-sized ones
    many = [torch.randn((int(r), 3), generator=g).to(torch.float16) for r in torch.randint(0, 9, (230,), generator=g)]
    got = kv_ops.concat_rows([s.to(DEV) for s in many])
    assert same_bits(got, torch.cat(many, 0))
    assert same_bits(got, orc.c_concat_rows(many))
    w = KVWorker(device=DEV)
    w.init_vecache()
    for i, s in enumerate(segs[:3]):
        w.write_vision_blocks(f"r{i}", s.to(DEV))
    assert same_bits(w.gather_vision_embeddings(["r0", "zz", "r2"]), torch.cat([segs[0], segs[2]], 0))
    assert w.gather_vision_embeddings(["r1"]) is w.extract_vision_blocks("r1")
    # the prepared segments follow the cache: an entry replaced through the dict itself, a non-contiguous
    # entry, a dropped entry, and a repeated gather
    repl = torch.randn((5, segs[0].shape[1]), generator=g).to(segs[0].dtype)
    w.ve_cache["r0"] = repl.to(DEV)
    wide = torch.randn((4, 2 * segs[0].shape[1]), generator=g).to(segs[0].dtype)
    w.ve_cache["r3"] = wide.to(DEV)[:, ::2]
    want = torch.cat([repl, segs[2], wide[:, ::2]], 0)
    for _ in range(2):
        assert same_bits(w.gather_vision_embeddings(["r0", "r2", "r3"]), want)
    del w.ve_cache["r2"]
    assert same_bits(w.gather_vision_embeddings(["r0", "r2", "r3"]), torch.cat([repl, wide[:, ::2]], 0))
    with pytest.raises(ValueError):
        w.ve_cache["bad"] = torch.zeros((2, 3), dtype=segs[0].dtype, device=DEV)
        w.gather_vision_embeddings(["r0", "bad"])


def test_concat_rows_non_contiguous_segments():
    say("vision concat: several non-contiguous segments of equal size (their contiguous copies must stay alive)")
    g = torch.Generator().manual_seed(15)
    wide = [torch.randn((256, 2 * 3584), generator=g).to(torch.bfloat16) for _ in range(6)]
    views = [w.to(DEV)[:, ::2] for w in wide]
    assert not views[0].is_contiguous()
    want = torch.cat([w[:, ::2] for w in wide], 0)
    for _ in range(3):
        got = kv_ops.concat_rows(views)
        assert same_bits(got, want)
        del got
    mixed = [views[0], wide[1].to(DEV)[:, :3584].contiguous(), views[2], views[3]]
    assert same_bits(kv_ops.concat_rows(mixed), torch.cat([wide[0][:, ::2], wide[1][:, :3584], wide[2][:, ::2],
                                                            wide[3][:, ::2]], 0))


def test_host_id_entry_points_match_the_device_table_ones():
    """emm_kv_pack_host_ids / emm_kv_unpack_host_ids carry the block table in the kernel argument block. Same
    bytes as the device-table entry points for tables of 1, 37, 512 (one launch's worth), 513 and 1300 ids
    (several launches), odd chunk sizes included; ids that the device path skips (negative, too large) are
    skipped; the Python layer picks the path by where the table lives."""
    import ctypes

    lib = _lib.load()
    L, NB = 3, 1400
    for block_shape, dtype in (((16, 4, 128), torch.bfloat16), ((3, 5), torch.float16), ((7,), torch.uint8)):
        g = torch.Generator().manual_seed(21)
        pool_c = [torch.randint(0, 255, (2, NB) + block_shape, generator=g).to(torch.uint8).view(torch.uint8)
                  for _ in range(L)]
        if dtype != torch.uint8:
            pool_c = [torch.randn((2, NB) + block_shape, generator=g).to(dtype) for _ in range(L)]
        pool_g = to_dev(pool_c)
        pv = PoolView(pool_g)
        for n in (1, 37, 512, 513, 1300):
            ids = torch.randperm(NB, generator=g)[:n]
            via_list = kv_ops.kv_pack(pv, ids.tolist())              # host table: argument-block path
            via_dev = kv_ops.kv_pack(pv, ids.to(DEV))                # device table
            assert same_bits(via_list, via_dev) and same_bits(via_list, orc.c_kv_pack(pool_c, ids.tolist()))
            d1 = [torch.full_like(p, 0) for p in pool_g]
            d2 = [torch.full_like(p, 0) for p in pool_g]
            dst_ids = torch.randperm(NB, generator=g)[:n]
            kv_ops.kv_unpack(PoolView(d1), dst_ids.tolist(), via_list)
            kv_ops.kv_unpack(PoolView(d2), dst_ids.to(DEV), via_list)
            assert same_bits(torch.stack(d1), torch.stack(d2))
    # the C ABI directly: skipped ids, the limit
    pool_g = to_dev(cpu_pool(2, 32, 16, 2, 64, torch.bfloat16, 5))
    pv = PoolView(pool_g)
    table = _lib.ptr_table(pv.ptrs)
    raw_ids = np.array([3, -1, 31, 32, 7, 10 ** 12], dtype=np.int64)
    out = torch.full(pv.packed_shape(6), 7.0, dtype=torch.bfloat16, device=DEV)
    rc = lib.emm_kv_pack_host_ids(table, 2, 2, 32, pv.chunk_bytes, raw_ids.ctypes.data, 6, out.data_ptr(),
                                  torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.emm_last_error()
    want = torch.full(pv.packed_shape(6), 7.0, dtype=torch.bfloat16)
    for l in range(2):
        for j, b in enumerate(raw_ids.tolist()):
            if 0 <= b < 32:
                want[l, :, j] = pool_g[l][:, b].cpu()
    assert same_bits(out, want)
    rc = lib.emm_kv_unpack_host_ids(table, 2, 2, 32, pv.chunk_bytes, None, 4, out.data_ptr(), None)
    assert rc == -1 and b"null" in lib.emm_last_error()



# ------------------------------------------------------------------ worker protocol
def make_pair(L=3, NB=32, bs=16, H=2, D=64, dtype=torch.bfloat16):
    link = LoopbackLink(world_size=2)
    src = KVWorker(0, DEV, bs, link, 0)
    dst = KVWorker(1, DEV, bs, link, 1)
    src.init_kvcache(NB, num_layers=L, num_kv_heads=H, head_size=D, dtype=dtype, monolithic=False)
    dst.init_kvcache(NB, num_layers=L, num_kv_heads=H, head_size=D, dtype=dtype, monolithic=True)
    g = torch.Generator().manual_seed(14)
    for t in src.kv_cache:
        t.copy_(torch.randn(t.shape, generator=g).to(dtype))
    for t in dst.kv_cache:
        t.fill_(-2.0)
    src.peers[1] = dst
    dst.peers[0] = src
    return src, dst


def check_moved(src, dst, si, di):
    src_c = [t.cpu() for t in src.kv_cache]
    want = [torch.full_like(t, -2.0) for t in src_c]
    orc.ref_write_kv_blocks(want, di, orc.ref_extract_kv_blocks(src_c, si))
    for l in range(len(want)):
        assert same_bits(dst.kv_cache[l], want[l])


def test_worker_p2p_send_recv():
    src, dst = make_pair()
    si, di = [5, 9, 0, 31], [1, 2, 3, 30]
    s = src.p2p_send_kv(1, si)
    per_layer = 2 * 4 * 16 * 2 * 64 * 2
    assert s == {"bytes": 3 * per_layer, "blocks": 4}
    r = dst.p2p_recv_kv(0, di)
    assert r == {"bytes": 3 * per_layer, "blocks": 4}
    check_moved(src, dst, si, di)
    # nothing pending -> error dict, not an exception
    r = dst.p2p_recv_kv(0, di)
    assert r["bytes"] == 0 and r["blocks"] == 0 and r["error"].startswith("NCCL recv failed: RuntimeError")
    bad = src.p2p_send_kv(1, [999])
    assert bad["bytes"] == 0 and bad["error"].startswith("NCCL send failed: IndexError")


def test_worker_coordinated_pull_and_collective():
    src, dst = make_pair()
    si, di = [7, 8, 30], [0, 15, 16]
    res = dst.p2p_coordinated_transfer_kv(src, 0, si, di)
    assert res["method"] == "coordinated_single_call" and res["blocks"] == 3 and res["bytes"] == 3 * 2 * 3 * 16 * 2 * 64 * 2
    check_moved(src, dst, si, di)
    res = dst.p2p_coordinated_transfer_kv(src, 0, si, di, timeout=-1.0)
    assert res["error"].startswith("Transfer timeout after -1.0s at layer 0/3")

    src, dst = make_pair()
    res = dst.p2p_pull_kv(0, si, di)
    assert res == {"bytes": 3 * 2 * 3 * 16 * 2 * 64 * 2, "blocks": 3}
    check_moved(src, dst, si, di)

    src, dst = make_pair()
    shape = (3, 2, 3, 16, 2, 64)
    a = src.collective_transfer_kv("g0", 0, si, shape, "torch.bfloat16", "send")
    b = dst.collective_transfer_kv("g0", 0, di, shape, "bf16", "recv")
    assert a == {"bytes": int(np.prod(shape)) * 2, "mode": "send"} and b["mode"] == "recv" and b["bytes"] == a["bytes"]
    check_moved(src, dst, si, di)
    with pytest.raises(ValueError, match="Unknown collective transfer mode"):
        src.collective_transfer_kv("g0", 0, si, shape, "bf16", "both")
    with pytest.raises(AssertionError, match="Block count mismatch"):
        dst.write_kv_blocks([1, 2], torch.zeros(shape, dtype=torch.bfloat16, device=DEV))


def test_failed_receive_leaves_no_stale_layers_on_the_link():
    """A receive that gives up (deadline, wrong block count) drops the rest of that transfer from the link:
    the next transfer between the same ranks moves its own bytes, not the stale layers."""
    src, dst = make_pair()
    si, di = [5, 9, 0, 31], [1, 2, 3, 30]
    # timeout before the first layer: the three queued layer messages must go away
    res = dst.p2p_coordinated_transfer_kv(src, 0, si, di, timeout=-1.0)
    assert "error" in res and src.link.pending(0, 1) == 0
    # wrong block count on the receiving side: error dict, link drained
    assert src.p2p_send_kv(1, si)["blocks"] == 4 and src.link.pending(0, 1) == 3
    bad = dst.p2p_recv_kv(0, di[:3])
    assert bad["bytes"] == 0 and "error" in bad and src.link.pending(0, 1) == 0
    # two sends queued, the first received with the wrong count: only the first is dropped
    si2, di2 = [7, 8, 30, 2], [0, 15, 16, 17]
    src.p2p_send_kv(1, si)
    src.p2p_send_kv(1, si2)
    assert "error" in dst.p2p_recv_kv(0, di[:2]) and src.link.pending(0, 1) == 3
    good = dst.p2p_recv_kv(0, di2)
    assert good["blocks"] == 4 and "error" not in good
    check_moved(src, dst, si2, di2)
    # pull: a request larger than the protocol's 1024 slots raises before anything is queued
    with pytest.raises(ValueError):
        dst.p2p_pull_kv(0, list(range(1025)), list(range(1025)))
    assert src.link.pending(1, 0, 999) == 0


def test_transfer_manager_moves_vision_embeddings():
    from elasticmm_amd.kv_transfer import KVTransferManager, TransferMethod

    src, dst = make_pair()
    src.init_vecache()
    dst.init_vecache()
    ve = torch.randn((300, 3584), generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    src.write_vision_blocks("img0", ve.to(DEV))
    m = KVTransferManager(TransferMethod.NCCL)
    m.register_workers("encoding", [src, dst], [0, 1])
    assert m.transfer_vision_embeddings_sync("img0", 0, [0, 1], 1, [4, 5]) is True
    assert same_bits(dst.extract_vision_blocks("img0"), ve)
    assert m.transfer_vision_embeddings_sync("absent", 0, [], 1, []) is False   # KeyError on the source -> False
    import asyncio
    assert asyncio.run(m.transfer_vision_embeddings("img0", 0, [0], 1, [1])) is True
    assert m.get_stats()["transfer_count"] == 2
    m.close()



# ------------------------------------------------------------------ full-size properties
def test_cfg2_full_size_migration_properties():
    """Qwen2-7B KV shape at full size: 28 x [2,60000,16,4,128] bf16 twice (2 x 51.3 GiB).
    Checked with torch's own device indexing as the second implementation."""
    L, NB, bs, H, D = 28, 60000, 16, 4, 128
    free, _ = torch.cuda.mem_get_info()
    need = 2 * L * 2 * NB * bs * H * D * 2 + (12 << 30)
    if free < need:
        # a full-size configuration that cannot run is a failure, not a skip: it must not go untested silently
        pytest.fail(f"this full-size configuration needs {need >> 30} GiB of free HBM, the device has {free >> 30} "
                    f"GiB free (an MI355X with nothing else on it has 288)", pytrace=False)
    say("cfg2 full size: allocating two 51.3 GiB pools")
    src = torch.empty((L, 2, NB, bs, H, D), dtype=torch.bfloat16, device=DEV)
    g = torch.Generator(device=DEV).manual_seed(2)
    for l in range(L):
        src[l].normal_(0.0, 0.5, generator=g)
    dst = torch.empty_like(src)
    dst.fill_(-1.0)
    gc = torch.Generator().manual_seed(2)
    nblk = [(int(p) + 1024 + 15) // 16 for p in torch.randint(512, 4097, (32,), generator=gc)]
    sperm = torch.randperm(NB, generator=gc)
    dperm = torch.randperm(NB, generator=gc)
    sp, dp = PoolView(src), PoolView(dst)
    off = 0
    tables = []
    for n in nblk:
        si, di = sperm[off:off + n].to(DEV), dperm[off:off + n].to(DEV)
        tables.append((si, di))
        off += n
        buf = kv_ops.kv_pack(sp, si)
        kv_ops.kv_unpack(dp, di, buf)
    torch.cuda.synchronize()
    say(f"cfg2 full size: moved {off} blocks, checking")
    moved = torch.zeros(NB, dtype=torch.bool, device=DEV)
    for r, (si, di) in enumerate(tables):
        moved[di] = True
        for l in range(0, L, 3) if r % 4 else range(L):
            ok = bool(torch.equal(dst[l][:, di], src[l][:, si]))
            assert ok, f"request {r} layer {l}"
    rest = (~moved).nonzero().squeeze(1)
    for l in range(L):
        ok = bool((dst[l][:, rest] == -1.0).all())
        assert ok, f"layer {l}: an untouched block changed"
    # batched form: one launch for all 32 requests
    dst.fill_(-1.0)
    all_si = torch.cat([t[0] for t in tables])
    all_di = torch.cat([t[1] for t in tables])
    kv_ops.kv_unpack(dp, all_di, kv_ops.kv_pack(sp, all_si))
    for l in (0, 13, 27):
        ok = bool(torch.equal(dst[l][:, all_di], src[l][:, all_si]))
        assert ok, f"batched: layer {l}"
    # copy_blocks inside the source pool: half of the used blocks to free blocks
    P = off // 2
    mapping = torch.stack([sperm[:P], sperm[off:off + P]], 1).to(DEV)
    before = src[5][:, mapping[:, 0]].clone()
    kv_ops.copy_blocks(sp, mapping)
    for l in (0, 5, 27):
        ok = bool(torch.equal(src[l][:, mapping[:, 1]], src[l][:, mapping[:, 0]]))
        assert ok, f"copy_blocks: layer {l}"
    ok = bool(torch.equal(src[5][:, mapping[:, 0]], before))
    assert ok, "copy_blocks changed a source block"
    del src, dst
    torch.cuda.empty_cache()


def test_cfg4_full_size_fp8_properties():
    """fp8 70B-class per-GPU shape at full size: 80 x [2,20000,16,8,128] e4m3 (52 GB per pool), 64 requests of
    1k-8k tokens. Byte moves are checked with torch's device indexing, the conversions against the CPU oracle on
    samples copied back."""
    L, NB, bs, H, D = 80, 20000, 16, 8, 128
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    need = 2 * L * 2 * NB * bs * H * D + (16 << 30)
    if free < need:
        # a full-size configuration that cannot run is a failure, not a skip: it must not go untested silently
        pytest.fail(f"this full-size configuration needs {need >> 30} GiB of free HBM, the device has {free >> 30} "
                    f"GiB free (an MI355X with nothing else on it has 288)", pytrace=False)
    say("cfg4 full size: two fp8 pools of 52 GB")
    g = torch.Generator().manual_seed(4)
    lens = torch.randint(1024, 8193, (64,), generator=g)
    nblk = [(int(t) + 15) // 16 for t in lens]
    total = sum(nblk)
    perm_s = torch.randperm(NB, generator=g)[:total].to(DEV)
    perm_d = torch.randperm(NB, generator=g)[:total].to(DEV)
    k_scales = torch.rand(L, generator=g) * 0.09 + 0.01
    v_scales = torch.rand(L, generator=g) * 0.09 + 0.01
    src = torch.empty((L, 2, NB, bs, H, D), dtype=torch.uint8, device=DEV)
    src.random_(0, 256)  # every byte value, NaN encodings included
    dst = torch.full_like(src, 0x5A)
    sp, dp = PoolView(src), PoolView(dst)
    off = 0
    tables = []
    for n in nblk:
        si, di = perm_s[off:off + n], perm_d[off:off + n]
        tables.append((si, di))
        kv_ops.kv_unpack(dp, di, kv_ops.kv_pack(sp, si))
        off += n
    torch.cuda.synchronize()
    say(f"cfg4 full size: moved {total} blocks, checking")
    for r, (si, di) in enumerate(tables):
        for l in range(r % 7, L, 7):
            ok = bool(torch.equal(dst[l][:, di], src[l][:, si]))
            assert ok, f"request {r} layer {l}"
    moved = torch.zeros(NB, dtype=torch.bool, device=DEV)
    moved[perm_d] = True
    rest = (~moved).nonzero().squeeze(1)
    for l in range(0, L, 5):
        ok = bool((dst[l][:, rest] == 0x5A).all())
        assert ok, f"layer {l}: an untouched block changed"
    del dst, dp
    torch.cuda.empty_cache()
    # quantising append of one step into all 80 layers with one launch
    T = 8448
    slots = make_slots(NB * bs, T, 4)
    gd = torch.Generator(device=DEV).manual_seed(4)
    keys = [(torch.randn((T, H, D), device=DEV, generator=gd) * 2).to(torch.bfloat16) for _ in range(L)]
    values = [(torch.randn((T, H, D), device=DEV, generator=gd) * 2).to(torch.bfloat16) for _ in range(L)]
    before = {l: src[l].cpu() for l in (0, 41, 79)}
    cache_ops.reshape_and_cache_flash_layers(keys, values, list(src.unbind(0)), slots.to(DEV), "fp8",
                                             k_scales.to(DEV), v_scales.to(DEV))
    for l, ref in before.items():
        orc.c_reshape_and_cache_fp8(keys[l].cpu(), values[l].cpu(), ref[0], ref[1], slots, float(k_scales[l]),
                                    float(v_scales[l]))
        assert same_bits(src[l], ref), f"fp8 append, layer {l}"
    del keys, values, before
    # dequantising unpack of the first 8 requests into a bf16 pool
    dq = torch.full((L, 2, NB, bs, H, D), -3.0, dtype=torch.bfloat16, device=DEV)
    dqp = PoolView(dq)
    for si, di in tables[:8]:
        kv_ops.kv_unpack_dequant_fp8(dqp, di, kv_ops.kv_pack(sp, si), k_scales, v_scales)
    torch.cuda.synchronize()
    for r in (0, 7):
        si, di = tables[r]
        for l in (0, 33, 79):
            for kv, sc in ((0, k_scales), (1, v_scales)):
                q = src[l][kv, si[:40]].cpu().numpy()
                got = dq[l][kv, di[:40]].cpu().view(torch.int16).numpy().view(np.uint16)
                want = orc.c_dequant_fp8(q, float(sc[l]), torch.bfloat16)
                assert (got == want).all(), f"dequant-unpack request {r} layer {l} kv {kv}"
    ok = bool((dq[17][:, rest[:2000]] == -3.0).all())
    assert ok, "dequant-unpack touched a block outside the tables"
    del src, sp, dq, dqp
    torch.cuda.empty_cache()


def test_cfg5_full_size_rebalance_properties():
    """Elastic rebalancing at full size: a 200 GB bf16 pool in the Qwen2-7B layout, copy_blocks of half of the live
    blocks to disjoint free blocks (54 500 pairs, 100 GB), with the vision-embedding gather of 128 images in between."""
    L, NB, bs, H, D = 28, 218000, 16, 4, 128
    torch.cuda.empty_cache()
    free, _ = torch.cuda.mem_get_info()
    need = L * 2 * NB * bs * H * D * 2 + (24 << 30)
    if free < need:
        # a full-size configuration that cannot run is a failure, not a skip: it must not go untested silently
        pytest.fail(f"this full-size configuration needs {need >> 30} GiB of free HBM, the device has {free >> 30} "
                    f"GiB free (an MI355X with nothing else on it has 288)", pytrace=False)
    say("cfg5 full size: one pool of 200 GB")
    pool = torch.empty((L, 2, NB, bs, H, D), dtype=torch.bfloat16, device=DEV)
    gd = torch.Generator(device=DEV).manual_seed(5)
    for l in range(L):
        pool[l].normal_(0.0, 0.5, generator=gd)
    g = torch.Generator().manual_seed(5)
    perm = torch.randperm(NB, generator=g)
    live, free_ids = perm[:NB // 2].to(DEV), perm[NB // 2:].to(DEV)
    for l in range(L):
        pool[l][:, free_ids] = -1.0  # canary in every free block
    P = live.numel() // 2
    mapping = torch.stack([live[:P], free_ids[:P]], 1).contiguous()
    sums = [pool[l][:, live].view(torch.int16).sum(dtype=torch.int64) for l in (0, 14, 27)]
    imgs = torch.randint(64, 2305, (128,), generator=g).tolist()
    embeds = [torch.randn((n, 3584), device=DEV, generator=gd).to(torch.bfloat16) for n in imgs]
    pv = PoolView(pool)
    eighth = P // 8
    cat = None
    for k in range(8):  # copy_blocks in eight slices with the vision gather in between
        hi = P if k == 7 else (k + 1) * eighth
        kv_ops.copy_blocks(pv, mapping[k * eighth:hi])
        if k == 3:
            cat = kv_ops.concat_rows(embeds)
    torch.cuda.synchronize()
    say("cfg5 full size: checking")
    for l in range(L):
        ok = bool(torch.equal(pool[l][:, mapping[:, 1]], pool[l][:, mapping[:, 0]]))
        assert ok, f"layer {l}: a destination differs from its source"
        ok = bool((pool[l][:, free_ids[P:]] == -1.0).all())
        assert ok, f"layer {l}: a free block outside the mapping changed"
    for l, s0 in zip((0, 14, 27), sums):
        ok = bool(pool[l][:, live].view(torch.int16).sum(dtype=torch.int64) == s0)
        assert ok, f"layer {l}: a live block changed"
    ok = bool(torch.equal(cat, torch.cat(embeds, 0)))
    assert ok, "vision gather differs from torch.cat"
    del pool, pv, embeds, cat
    torch.cuda.empty_cache()


# ------------------------------------------------------------------ prepared plan / HIP graph
def test_layered_append_plan_reuse_and_graph_replay():
    """A prepared whole-step append is reused with new data and new slots, and the per-layer
    appends replayed from a captured HIP graph give the eager result on every replay (the
    program's own eager work and synchronisations run between the replays)."""
    NB, bs, H, D, T, L = 64, 16, 4, 128, 300, 3
    g = torch.Generator().manual_seed(15)
    keys = [torch.zeros((T, H, D), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    values = [torch.zeros((T, H, D), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    slots_g = torch.zeros(T, dtype=torch.long, device=DEV)
    pool_plan = [torch.zeros((2, NB, bs, H, D), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    pool_graph = [torch.zeros((2, NB, bs, H, D), dtype=torch.bfloat16, device=DEV) for _ in range(L)]
    pool_c = [torch.zeros((2, NB, bs, H, D), dtype=torch.bfloat16) for _ in range(L)]
    plan = cache_ops.layered_append(keys, values, pool_plan, "auto")

    def per_layer():
        for l in range(L):
            cache_ops.reshape_and_cache_flash(keys[l], values[l], pool_graph[l][0], pool_graph[l][1], slots_g, "auto")

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        per_layer()                      # warm-up outside capture
    torch.cuda.current_stream().wait_stream(side)
    for p in pool_graph:
        p.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        per_layer()
    for it in range(4):
        slots = make_slots(NB * bs, T, 100 + it, pad_frac=0.1)
        slots_g.copy_(slots)
        for l in range(L):
            k = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
            v = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
            keys[l].copy_(k)
            values[l].copy_(v)
            orc.c_reshape_and_cache(k, v, pool_c[l][0], pool_c[l][1], slots)
        plan(slots_g)
        graph.replay()
        torch.cuda.synchronize()
        # unrelated eager work between replays
        junk = kv_ops.kv_pack(PoolView(pool_plan), [1, 2, 3])
        assert junk.shape[2] == 3
        for l in range(L):
            assert same_bits(pool_plan[l], pool_c[l]), f"plan, iteration {it}, layer {l}"
            assert same_bits(pool_graph[l], pool_c[l]), f"graph replay {it}, layer {l}"


def test_migration_step_replayed_from_a_hip_graph():
    """pack -> unpack -> fused migrate -> copy_blocks -> paged append -> vision gather captured once in a HIP
    graph over fixed buffers and device-resident tables; every replay (new tables, new data, eager work and
    synchronisations in between) must equal the oracle."""
    L, NB, bs, H, D, n, T = 3, 48, 16, 2, 64, 9, 40
    g = torch.Generator().manual_seed(23)
    src_c = cpu_pool(L, NB, bs, H, D, torch.bfloat16, 23)
    src = to_dev(src_c)
    dst = [torch.zeros_like(t) for t in src]
    mig = [torch.zeros_like(t) for t in src]
    sp, dp, mp = PoolView(src), PoolView(dst), PoolView(mig)
    si = torch.zeros(n, dtype=torch.long, device=DEV)
    di = torch.zeros(n, dtype=torch.long, device=DEV)
    mapping = torch.zeros((4, 2), dtype=torch.long, device=DEV)
    buf = torch.empty(sp.packed_shape(n), dtype=torch.bfloat16, device=DEV)
    key = torch.zeros((T, H, D), dtype=torch.bfloat16, device=DEV)
    value = torch.zeros_like(key)
    slots_g = torch.zeros(T, dtype=torch.long, device=DEV)
    kc = torch.zeros((NB, H, D // 8, bs, 8), dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros((NB, H, D, bs), dtype=torch.bfloat16, device=DEV)
    segs = [torch.zeros((r, 24), dtype=torch.bfloat16, device=DEV) for r in (5, 1, 7)]
    sources = [kv_ops.RowSource(t) for t in segs]
    cat = torch.empty((13, 24), dtype=torch.bfloat16, device=DEV)

    def step():
        kv_ops.kv_pack(sp, si, out=buf)
        kv_ops.kv_unpack(dp, di, buf)
        kv_ops.kv_migrate(sp, si, mp, di)
        kv_ops.copy_blocks(dp, mapping)
        cache_ops.reshape_and_cache(key, value, kc, vc, slots_g, "auto")
        kv_ops.concat_row_sources(sources, out=cat)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    for t in (*dst, *mig, kc, vc):
        t.zero_()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step()
    dst_c = [torch.zeros_like(t) for t in src_c]
    mig_c = [torch.zeros_like(t) for t in src_c]
    kc_c, vc_c = torch.zeros(kc.shape, dtype=torch.bfloat16), torch.zeros(vc.shape, dtype=torch.bfloat16)
    for it in range(4):
        perm = torch.randperm(NB, generator=g)
        s_tab, d_tab = perm[:n], torch.randperm(NB, generator=g)[:n]
        free = [b for b in range(NB) if b not in set(d_tab.tolist())]
        pairs = torch.tensor([[int(d_tab[i]), free[i + it]] for i in range(4)])
        slots = make_slots(NB * bs, T, 200 + it, pad_frac=0.1)
        k = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
        v = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
        new_segs = [torch.randn(t.shape, generator=g).to(torch.bfloat16) for t in segs]
        si.copy_(s_tab)
        di.copy_(d_tab)
        mapping.copy_(pairs)
        slots_g.copy_(slots)
        key.copy_(k)
        value.copy_(v)
        for t, c in zip(segs, new_segs):
            t.copy_(c)
        graph.replay()
        torch.cuda.synchronize()
        packed = orc.ref_extract_kv_blocks(src_c, s_tab.tolist())
        orc.ref_write_kv_blocks(dst_c, d_tab.tolist(), packed)
        orc.ref_write_kv_blocks(mig_c, d_tab.tolist(), packed)
        orc.ref_copy_blocks(dst_c, pairs)
        orc.c_reshape_and_cache_paged(k, v, kc_c, vc_c, slots)
        assert same_bits(buf, packed), f"replay {it}: pack"
        for l in range(L):
            assert same_bits(dst[l], dst_c[l]), f"replay {it}: unpack + copy_blocks, layer {l}"
            assert same_bits(mig[l], mig_c[l]), f"replay {it}: migrate, layer {l}"
        assert same_bits(kc, kc_c) and same_bits(vc, vc_c), f"replay {it}: paged append"
        assert same_bits(cat, torch.cat(new_segs, 0)), f"replay {it}: vision gather"
        junk = kv_ops.kv_pack(sp, [0, 1])  # unrelated eager work between the replays
        assert junk.shape[2] == 2


def test_large_block_count_splits_launches():
    """More than 65 535 blocks in one call (the grid's y limit): tiny chunks keep it small."""
    NB, n = 70000, 66000
    g = torch.Generator().manual_seed(16)
    src_c = [torch.randint(0, 255, (2, NB, 1, 1, 16), generator=g, dtype=torch.uint8)]
    si = torch.randperm(NB, generator=g)[:n]
    di = torch.randperm(NB, generator=g)[:n]
    src_g = to_dev(src_c)
    buf = kv_ops.kv_pack(PoolView(src_g), si.to(DEV))
    assert same_bits(buf, orc.c_kv_pack(src_c, si.numpy()))
    dst_g = [torch.zeros_like(src_g[0])]
    kv_ops.kv_unpack(PoolView(dst_g), di.to(DEV), buf)
    dst_c = [torch.zeros_like(src_c[0])]
    orc.c_kv_unpack(dst_c, di.numpy(), raw(buf))
    assert same_bits(dst_g[0], dst_c[0])
    dst2 = [torch.zeros_like(src_g[0])]
    kv_ops.kv_migrate(PoolView(src_g), si.to(DEV), PoolView(dst2), di.to(DEV))
    assert same_bits(dst2[0], dst_c[0])
    mapping = torch.stack([si[:33000], di[:33000]], 1)
    free_dst = torch.tensor(sorted(set(range(NB)) - set(si.tolist()))[:4000])
    mapping = torch.stack([si[:4000], free_dst], 1).contiguous()
    cp_g = to_dev(src_c)
    kv_ops.copy_blocks(PoolView(cp_g), mapping.to(DEV))
    cp_c = [src_c[0].clone()]
    orc.c_copy_blocks(cp_c, mapping.numpy())
    assert same_bits(cp_g[0], cp_c[0])
    # dequantising unpack with more than 65 535 blocks
    dq_g = [torch.zeros((2, NB, 1, 1, 16), dtype=torch.bfloat16, device=DEV)]
    dq_c = [torch.zeros((2, NB, 1, 1, 16), dtype=torch.bfloat16)]
    kv_ops.kv_unpack_dequant_fp8(PoolView(dq_g), di.to(DEV), buf, [0.05], [0.07])
    orc.c_unpack_dequant_fp8(dq_c, di.numpy(), raw(buf), [0.05], [0.07])
    assert same_bits(dq_g[0], dq_c[0])


# ------------------------------------------------------------------ GPU <-> CPU swap
def test_swap_blocks_out_and_in():
    L, NB, NBC, bs, H, D = 3, 24, 10, 16, 2, 64
    w = KVWorker(0, DEV, bs)
    w.init_kvcache(NB, NBC, num_layers=L, num_kv_heads=H, head_size=D, dtype=torch.bfloat16)
    assert len(w.kv_swap) == L and w.kv_swap[0].is_pinned() and tuple(w.kv_swap[0].shape) == (2, NBC, bs, H, D)
    g = torch.Generator().manual_seed(17)
    gpu_c = [torch.randn((2, NB, bs, H, D), generator=g).to(torch.bfloat16) for _ in range(L)]
    for t, c in zip(w.kv_cache, gpu_c):
        t.copy_(c)
    for t in w.kv_swap:
        t.fill_(-4.0)
    torch.cuda.synchronize()
    src_gpu, dst_cpu = [5, 17, 2, 23], [9, 0, 4, 1]
    w.swap_blocks(["r1", "r2"], src_gpu, dst_cpu, is_swap_in=False)
    w.wait_for_all_swap_out()
    torch.cuda.synchronize()
    cpu_want = [torch.full((2, NBC, bs, H, D), -4.0, dtype=torch.bfloat16) for _ in range(L)]
    for l in range(L):
        cpu_want[l][:, dst_cpu] = gpu_c[l][:, src_gpu]
        assert same_bits(w.kv_swap[l], cpu_want[l]), f"swap-out layer {l}"
        assert same_bits(w.kv_cache[l], gpu_c[l])
    # swap the same blocks back in under other GPU block ids; ordered after the swap-out by r1's event
    back = [20, 21, 22, 0]
    w.swap_blocks(["r1"], dst_cpu, back, is_swap_in=True)
    w.wait_for_all_swap_in()
    torch.cuda.synchronize()
    for l in range(L):
        want = gpu_c[l].clone()
        want[:, back] = gpu_c[l][:, src_gpu]
        assert same_bits(w.kv_cache[l], want), f"swap-in layer {l}"
    assert set(w.swap_event_table) == {"r1", "r2"}
    w.clear_request_resource("r1")
    assert set(w.swap_event_table) == {"r2"}
    with pytest.raises(ValueError, match="Block count mismatch"):
        w.swap_blocks(["r1"], [1, 2], [3], True)
    with pytest.raises(IndexError):
        w.swap_blocks(["r1"], [NBC], [3], True)
    fresh = KVWorker(0, DEV, bs)
    with pytest.raises(RuntimeError, match="not initialized"):
        fresh.swap_blocks(["r"], [0], [0], True)


def test_block_manager_drives_a_swap_cycle():
    """Requests are swapped out by the block manager, their GPU blocks are reused and overwritten by another
    request, and after the swap-in every request's blocks hold its own data again (block ids differ)."""
    L, NB, NBC, bs, H, D = 2, 12, 12, 16, 2, 32
    w = KVWorker(0, DEV, bs)
    w.init_kvcache(NB, NBC, num_layers=L, num_kv_heads=H, head_size=D, dtype=torch.float16)
    bm = BlockManager(NB, block_size=bs, max_num_cpu_blocks=NBC, workers=[w])
    g = torch.Generator().manual_seed(29)
    data = {}

    def fill(rid, nblocks):
        table = bm.allocate_blocks(rid, nblocks)
        data[rid] = torch.randn((L, 2, nblocks, bs, H, D), generator=g).to(torch.float16)
        w.write_kv_blocks(table, data[rid].to(DEV))

    def check(rid):
        assert bm.get_location(rid) == BlockLocation.GPU
        assert same_bits(w.extract_kv_blocks(bm.get_block_table(rid)), data[rid]), rid

    fill("a", 5)
    fill("b", 4)
    fill("c", 3)
    bm.swap_out_requests(["a", "b"])
    assert bm.get_location("a") == BlockLocation.CPU and bm.get_block_table("c") == [9, 10, 11]
    fill("d", 8)            # needs the blocks of a and b: the manager waits for the swap-out first
    assert set(bm.get_block_table("d")) <= set(range(9))
    check("c")
    check("d")
    bm.free_blocks("d")
    bm.swap_in_requests(["b", "a"])
    bm.wait_for_all_swap_in()
    for rid in ("a", "b", "c"):
        check(rid)
    assert sorted(bm.get_block_table("a") + bm.get_block_table("b") + bm.get_block_table("c")) == \
        sorted(set(bm.get_block_table("a") + bm.get_block_table("b") + bm.get_block_table("c")))
    bm.clear_request_resource_batched(["a", "b"])
    assert not w.swap_event_table


def test_fp8_append_scale_range_paths():
    """Extreme and awkward scales (powers of two far from 1, all-ones mantissas, a negative
    scale, the smallest normal and the largest finite float): the quotient must be the one
    correctly rounded fp32 division of the oracle for every bf16 and f16 input."""
    import struct

    def f32(bits):
        return struct.unpack("<f", struct.pack("<I", bits))[0]

    scales = [2.0 ** -30, 2.0 ** 30, 2.0 ** -31, 2.0 ** 31, 3.0e10, 1.0e-12, f32(0x3DFFFFFF), f32(0x3C7FFFFF),
              f32(0x3F7FFFFF), -0.05, 0.013671875, 1.0 / 3.0, 448.0, f32(0x00800000), f32(0x7F7FFFFF)]
    slots = torch.arange(64, device=DEV)
    for dtype in (torch.bfloat16, torch.float16):
        allx = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
        key = allx.view(64, 8, 128).to(DEV)
        for s in scales:
            s32 = float(np.float32(s))
            kc = torch.zeros((4, 16, 8, 128), dtype=torch.uint8, device=DEV)
            vc = torch.zeros_like(kc)
            sc = torch.tensor([s32], dtype=torch.float32, device=DEV)
            cache_ops.reshape_and_cache_flash(key, key, kc, vc, slots, "fp8", sc, sc)
            got = raw(kc)
            want = orc.c_quant_fp8(allx, s32).reshape(-1)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, f"{dtype} scale {s32!r}: {bad.size} mismatches, first input bits {bad[:6].tolist()} " \
                                  f"got {got[bad[:6]].tolist()} want {want[bad[:6]].tolist()}"
            assert (raw(vc) == want).all()


def test_fp8_quantise_many_scales_against_the_division():
    """The append divides through a reciprocal and one correction step wherever 2^-30 <= |scale| <= 2^30.
    Scales whose significands are the known hard cases of that scheme (all ones, all ones minus a few ulps, one ulp
    above a power of two, around 1.5, alternating bits) at every third exponent of the range, plus 320 random
    scales: every bf16 and f16 input must give the byte of the oracle's correctly rounded division."""
    import struct

    def f32(bits):
        return struct.unpack("<f", struct.pack("<I", bits))[0]

    mantissas = [0, 1, 2, 3, 0x7FFFFF, 0x7FFFFE, 0x7FFFFD, 0x400000, 0x400001, 0x3FFFFF, 0x555555, 0x2AAAAA]
    scales = [f32(((127 + e) << 23) | m) for e in range(-30, 30, 3) for m in mantissas]
    rng = np.random.default_rng(11)
    scales += [f32(int(b)) for b in rng.integers((127 - 30) << 23, (127 + 30) << 23, 320)]
    scales = [s for s in scales if 2.0 ** -30 <= s <= 2.0 ** 30]
    slots = torch.arange(64, device=DEV)
    group = 80
    for dtype in (torch.bfloat16, torch.float16):
        allx = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
        key = allx.view(64, 8, 128).to(DEV)
        for g0 in range(0, len(scales), group):
            part = scales[g0:g0 + group]
            L = len(part)
            pools = [torch.zeros((2, 4, 16, 8, 128), dtype=torch.uint8, device=DEV) for _ in range(L)]
            sc = torch.tensor(part, dtype=torch.float32)
            cache_ops.reshape_and_cache_flash_layers([key] * L, [key] * L, pools, slots, "fp8", sc, sc)
            for l, sv in enumerate(part):
                want = orc.c_quant_fp8(allx, float(np.float32(sv))).reshape(-1)
                got = raw(pools[l][0])
                bad = np.nonzero(got != want)[0]
                assert bad.size == 0, f"{dtype} scale {sv!r}: {bad.size} mismatches, first input bits " \
                                      f"{bad[:6].tolist()} got {got[bad[:6]].tolist()} want {want[bad[:6]].tolist()}"
                assert (raw(pools[l][1]) == want).all()


def test_fp8_saturating_mode_exhaustive_on_gpu():
    """kv_cache_dtype "fp8_e4m3_sat": every bf16 and f16 input at the golden scales, extreme scales that
    take the division path, and a negative scale, through the flash append (vector and element paths), the
    whole-step launch and the paged layout, against the oracle's clamp-then-cast. NaN inputs stay NaN,
    overflow and infinities give +-448."""
    import struct

    def f32(bits):
        return struct.unpack("<f", struct.pack("<I", bits))[0]

    kat = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "fp8_kat.json")))
    scales = list(kat["scales"]) + [2.0 ** -31, 2.0 ** 31, -0.05, f32(0x3DFFFFFF), 448.0]
    slots = torch.arange(64, device=DEV)
    for dtype in (torch.bfloat16, torch.float16):
        allx = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
        key = allx.view(64, 8, 128).to(DEV)
        for sv in scales:
            s32 = float(np.float32(sv))
            want = orc.c_quant_fp8_sat(allx, s32).reshape(-1)
            sc = torch.tensor([s32], dtype=torch.float32, device=DEV)
            kc = torch.zeros((4, 16, 8, 128), dtype=torch.uint8, device=DEV)
            vc = torch.zeros_like(kc)
            cache_ops.reshape_and_cache_flash(key, key, kc, vc, slots, "fp8_e4m3_sat", sc, sc)
            got = raw(kc)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, f"{dtype} scale {s32!r}: {bad.size} mismatches, first input bits {bad[:6].tolist()} " \
                                  f"got {got[bad[:6]].tolist()} want {want[bad[:6]].tolist()}"
            assert (raw(vc) == want).all()
        # the other entry points at one scale: whole-step launch, element-wise path (rows of 7 elements),
        # paged layout
        s32 = float(np.float32(0.037))
        want = orc.c_quant_fp8_sat(allx, s32).reshape(-1)
        sc = torch.tensor([s32], dtype=torch.float32, device=DEV)
        pools = [torch.zeros((2, 4, 16, 8, 128), dtype=torch.uint8, device=DEV) for _ in range(2)]
        cache_ops.reshape_and_cache_flash_layers([key, key], [key, key], pools, slots, "fp8_sat", [s32, s32], [s32, s32])
        assert (raw(pools[1][0]) == want).all() and (raw(pools[0][1]) == want).all()
        odd = allx[:7 * 9360].view(9360, 1, 7).to(DEV)
        kc7 = torch.zeros((585, 16, 1, 7), dtype=torch.uint8, device=DEV)
        vc7 = torch.zeros_like(kc7)
        cache_ops.reshape_and_cache_flash(odd, odd, kc7, vc7, torch.arange(9360, device=DEV), "fp8_e4m3_sat", sc, sc)
        assert (raw(kc7) == want[:7 * 9360]).all()
        kcp = torch.zeros((4, 8, 128 // 16, 16, 16), dtype=torch.uint8, device=DEV)
        vcp = torch.zeros((4, 8, 128, 16), dtype=torch.uint8, device=DEV)
        cache_ops.reshape_and_cache(key, key, kcp, vcp, slots, "fp8_e4m3_sat", sc, sc)
        # value_cache[b, h, d, o] = q(value[t, h, d]) with t = b * 16 + o
        assert (raw(vcp.permute(0, 3, 1, 2).contiguous()) == want).all()
        assert (raw(kcp.permute(0, 3, 1, 2, 4).contiguous()) == want).all()


def test_fp8_fast_quotient_equals_the_division_for_every_significand_pair():
    """The append divides through a reciprocal and one correction step. That the result is the correctly rounded
    quotient is established by exhaustion: the three operations commute with powers of two while everything stays
    in the normal range, so only the significands matter — all 2^10 x significands (the 11 significant bits of an
    f16; bf16 values are a subset), both signs, against all 2^23 scale significands, 1.7e10 pairs per exponent
    pair. Several exponent pairs are swept: quotients in the middle of the fp8 range, at its overflow edge and in
    its subnormal range, and scales at both ends of the interval the fast form is used in. Every fp32 quotient
    must equal the division's, and the bytes after conversion too, in both overflow modes."""
    hooks = _lib.load_hooks()
    pairs = [(0, 0), (3, -5), (-2, -4), (4, -5), (-12, -5), (-3, -30), (5, 30), (2, -7)]
    for x_exp, s_exp in pairs:
        counters = torch.zeros(5, dtype=torch.int64, device=DEV)
        rc = hooks.emm_hook_fp8_quotient_sweep(x_exp, s_exp, 0, 1 << 23, counters.data_ptr(),
                                               torch.cuda.current_stream().cuda_stream)
        assert rc == 0, hooks.emm_last_error()
        c = counters.cpu().tolist()
        say(f"quotient sweep x_exp={x_exp} s_exp={s_exp}: {c[3]} pairs, raw mismatches {c[0]}, byte mismatches {c[1]} / {c[2]}")
        assert c[3] == 2048 * (1 << 23)
        assert c[0] == 0 and c[1] == 0 and c[2] == 0, f"x_exp={x_exp} s_exp={s_exp}: first differing pair {c[4]:#x}"
    # outside the interval the library takes the division itself: the sweep then compares it with itself and
    # still has to report a clean run (keeps the hook honest about which path it exercised)
    counters = torch.zeros(5, dtype=torch.int64, device=DEV)
    assert hooks.emm_hook_fp8_quotient_sweep(0, 40, 0, 1 << 12, counters.data_ptr(),
                                             torch.cuda.current_stream().cuda_stream) == 0
    assert counters.cpu().tolist()[:4] == [0, 0, 0, 2048 * (1 << 12)]



# ------------------------------------------------------------------ transfer manager on real workers
def test_transfer_manager_methods_move_the_same_bytes():
    from elasticmm_amd.kv_transfer import KVTransferManager, TransferMethod

    si, di = [3, 30, 7, 12], [0, 1, 29, 15]
    for method, batching in ((TransferMethod.P2P_COPY, False), (TransferMethod.NCCL, False),
                             (TransferMethod.CUDA_IPC, False), (TransferMethod.STAGED_COPY, False),
                             (TransferMethod.NCCL, True)):
        src, dst = make_pair()
        m = KVTransferManager(method, enable_batching=batching, batch_size=2, batch_timeout=1e9)
        m.register_workers("prefill", [src], [0])
        m.register_workers("decoding", [dst], [1])
        if batching:
            assert m.transfer_kv_cache_sync("a", 0, 1, si[:2], di[:2]) is True
            assert m.transfer_kv_cache_sync("b", 0, 1, si[2:], di[2:]) is True     # reaches the batch size: flush
            assert m.get_stats()["transfer_count"] == 2
        else:
            assert m.transfer_kv_cache_sync("a", 0, 1, si, di) is True
        torch.cuda.synchronize()
        check_moved(src, dst, si, di)
        assert m.transfer_kv_cache_sync("bad", 0, 1, [999], [0]) is (True if batching else False)


def test_migration_manager_moves_blocks_and_vision_embeddings():
    """The (stage, worker id)-addressed manager: KV blocks and a request's vision embeddings move from the
    prefill worker to the decoding worker; an unknown worker or a bad block id reports failure."""
    import asyncio
    from elasticmm_amd.kv_transfer import KVMigrationManager

    si, di = [3, 30, 7, 12], [0, 1, 29, 15]
    src, dst = make_pair()
    m = KVMigrationManager()
    assert m.migrate_kv_blocks_sync("a", "prefill", 0, si, "decoding", 0, di) is False  # nobody registered
    m.register_worker("prefill", 0, src)
    m.register_worker("Decoding", 0, dst)
    assert asyncio.run(m.migrate_kv_blocks("a", "prefill", 0, si, "decoding", 0, di)) is True
    torch.cuda.synchronize()
    check_moved(src, dst, si, di)
    assert m.migrate_kv_blocks_sync("bad", "prefill", 0, [999], "decoding", 0, [0]) is False
    src.init_vecache()
    dst.init_vecache()
    e = torch.randn((11, 64), device=DEV)
    src.write_vision_blocks("a", e)
    assert asyncio.run(m.migrate_vision_embeddings("a", "prefill", 0, "decoding", 0)) is True
    assert dst.get_ve_shape("a") == (11, 64) and dst.extract_vision_blocks("a") is e
    assert m.migrate_vision_embeddings_sync("missing", "prefill", 0, "decoding", 0) is False
    assert m.get_stats()["migration_count"] == 2
    m.unregister_worker("prefill", 0)
    assert m.migrate_kv_blocks_sync("a", "prefill", 0, si, "decoding", 0, di) is False


def test_migrate_requests_between_two_workers():
    """Elastic rescheduling of whole requests: destination tables come from the destination's block manager,
    the blocks move through each transfer method, the source blocks are freed afterwards; a destination that is
    too small leaves both sides as they were."""
    from elasticmm_amd.kv_transfer import KVTransferManager, TransferMethod

    for method, batching in ((TransferMethod.P2P_COPY, False), (TransferMethod.NCCL, False),
                             (TransferMethod.CUDA_IPC, False), (TransferMethod.NCCL, True)):
        src, dst = make_pair()
        NB = src.pool.num_blocks
        src_bm, dst_bm = BlockManager(NB), BlockManager(NB)
        dst_bm.allocate_blocks("resident", 5)                 # destination tables start at block 5
        for rid, n in (("skip-me", 2), ("a", 4), ("b", 3), ("c", 6)):
            src_bm.allocate_blocks(rid, n)
        src_bm.free_blocks("skip-me")
        tables = {r: list(src_bm.get_block_table(r)) for r in ("a", "b", "c")}
        before = [t.clone() for t in src.kv_cache]
        m = KVTransferManager(method, enable_batching=batching, batch_size=2, batch_timeout=1e9)
        m.register_workers("prefill", [src], [0])
        m.register_workers("decoding", [dst], [1])
        assert m.migrate_requests_sync(["a", "skip-me", "b", "c"], 0, src_bm, 1, dst_bm) is True
        torch.cuda.synchronize()
        for r, si in tables.items():
            di = dst_bm.get_block_table(r)
            assert len(di) == len(si) and min(di) >= 5
            for l in range(len(before)):
                ok = bool(torch.equal(dst.kv_cache[l][:, di], before[l][:, si]))
                assert ok, f"{method} batching={batching}: request {r} layer {l}"
            assert src_bm.get_block_table(r) == []
        assert src_bm.get_num_avail_gpu_blocks() == NB
        moved = sum(len(t) for t in tables.values())
        assert dst_bm.get_num_avail_gpu_blocks() == NB - 5 - moved
        # too large for what is left on the destination
        src_bm.allocate_blocks("huge", NB - 2)
        assert m.migrate_requests_sync(["huge"], 0, src_bm, 1, dst_bm) is False
        assert len(src_bm.get_block_table("huge")) == NB - 2 and dst_bm.get_block_table("huge") == []


def test_migration_coroutine_is_ordered_with_the_callers_side_stream():
    """A caller that works on a side stream: it fills the source blocks with a long kernel chain on that stream,
    awaits ``migrate_requests`` inside ``torch.cuda.stream(side)``, and overwrites the (freed) source blocks on
    the same stream right afterwards, never synchronising in between. The transfer is launched on the caller's
    current stream, so the pack sees the filled blocks and the overwrite cannot overtake it — for the methods
    that do not synchronise the device themselves (P2P_COPY, CUDA_IPC)."""
    import asyncio

    from elasticmm_amd.kv_transfer import KVMigrationManager, KVTransferManager, TransferMethod

    for method in (TransferMethod.P2P_COPY, TransferMethod.CUDA_IPC):
        src, dst = make_pair(L=6, NB=600, bs=16, H=4, D=128)
        NB = src.pool.num_blocks
        src_bm, dst_bm = BlockManager(NB), BlockManager(NB)
        dst_bm.allocate_blocks("resident", 7)
        for rid, n in (("a", 200), ("b", 150)):
            src_bm.allocate_blocks(rid, n)
        tables = {r: list(src_bm.get_block_table(r)) for r in ("a", "b")}
        m = KVTransferManager(method)
        m.register_workers("prefill", [src], [0])
        m.register_workers("decoding", [dst], [1])
        side = torch.cuda.Stream()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            for t in src.kv_cache:            # queued on the side stream only; still running when the pack is queued
                for _ in range(4):
                    t.normal_()
                t.mul_(0.5)
            ok = asyncio.run(m.migrate_requests(["a", "b"], 0, src_bm, 1, dst_bm))
            want = [t.clone() for t in src.kv_cache]     # what the pack must have seen
            for t in src.kv_cache:            # the source blocks are free now: the caller reuses them at once
                t.zero_()
        side.synchronize()
        assert ok is True
        for r, si in tables.items():
            di = dst_bm.get_block_table(r)
            for l in range(len(want)):
                assert torch.equal(dst.kv_cache[l][:, di], want[l][:, si]), f"{method}: request {r} layer {l}"
        # the (stage, worker id) manager the same way
        mm = KVMigrationManager()
        mm.register_worker("prefill", 0, src)
        mm.register_worker("decoding", 0, dst)
        with torch.cuda.stream(side):
            for t in src.kv_cache:
                t.normal_()
            ok = asyncio.run(mm.migrate_kv_blocks("x", "prefill", 0, [1, 2, 3], "decoding", 0, [9, 8, 7]))
            want = [t.clone() for t in src.kv_cache]
            for t in src.kv_cache:
                t.zero_()
        side.synchronize()
        assert ok is True
        for l in range(len(want)):
            assert torch.equal(dst.kv_cache[l][:, [9, 8, 7]], want[l][:, [1, 2, 3]])


def test_step_from_block_tables_to_both_cache_layouts():
    """Block manager -> slot mapping -> append: a step of two prompts and two decode tokens lands where the
    tables say, in the flash layout and in the paged-attention layout."""
    NB, bs, H, D = 40, 16, 2, 64
    bm = BlockManager(NB, block_size=bs)
    lens = {"p0": 70, "p1": 33, "d0": 21, "d1": 48}
    for rid, n in lens.items():
        bm.allocate_blocks(rid, bm.get_num_blocks_needed(n))
    bm.free_blocks("p0")
    bm.allocate_blocks("p0", bm.get_num_blocks_needed(70))          # tables are no longer in block order
    order = ["p0", "d0", "p1", "d1"]
    ctx = [0, 20, 0, 47]
    q = [70, 1, 33, 1]
    tables = [bm.get_block_table(r) for r in order]
    slots = cache_ops.compute_slot_mapping(tables, ctx, q, bs, pad_to=112, device=DEV)
    T = 112
    g = torch.Generator().manual_seed(37)
    key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    kc = torch.zeros((NB, bs, H, D), dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    kc_g, vc_g = kc.to(DEV), vc.to(DEV)
    cache_ops.reshape_and_cache_flash(key.to(DEV), value.to(DEV), kc_g, vc_g, slots, "auto")
    orc.c_reshape_and_cache(key, value, kc, vc, slots.cpu())
    assert same_bits(kc_g, kc) and same_bits(vc_g, vc)
    ok = bool(torch.equal(kc_g[tables[0][4], 5].cpu(), key[69]))     # last token of p0: position 69 = block 4, offset 5
    assert ok
    ok = bool(torch.equal(kc_g[tables[3][2], 15].cpu(), key[104]))   # d1's token (index 70 + 1 + 33) at position 47
    assert ok
    assert int((slots < 0).sum()) == 7
    kp = torch.zeros((NB, H, D // 8, bs, 8), dtype=torch.bfloat16)
    vp = torch.zeros((NB, H, D, bs), dtype=torch.bfloat16)
    kp_g, vp_g = kp.to(DEV), vp.to(DEV)
    cache_ops.reshape_and_cache(key.to(DEV), value.to(DEV), kp_g, vp_g, slots, "auto")
    orc.c_reshape_and_cache_paged(key, value, kp, vp, slots.cpu())
    assert same_bits(kp_g, kp) and same_bits(vp_g, vp)
    assert same_bits(kp_g, kc_g.view(NB, bs, H, D // 8, 8).permute(0, 2, 3, 1, 4).contiguous())


def test_spread_allocation_of_a_pool():
    """A pool whose layers are allocated in stripes spread over the device memory: same list API, layers
    disjoint, consecutive layers in different stripes (where the stripes land physically cannot be seen from here), and the kernels give the oracle's bytes on it."""
    from elasticmm_amd.worker import allocate_layers_spread

    L, NB, bs, H, D = 7, 4096, 16, 2, 64       # 32 MiB per layer: large enough to be allocations of their own
    torch.cuda.empty_cache()
    w = KVWorker(0, DEV, bs)
    w.init_kvcache(NB, num_layers=L, num_kv_heads=H, head_size=D, dtype=torch.bfloat16, spread_stripes=3)
    assert len(w.kv_cache) == L and all(tuple(t.shape) == (2, NB, bs, H, D) and t.is_contiguous() for t in w.kv_cache)
    nbytes = w.kv_cache[0].numel() * 2
    spans = sorted((t.data_ptr(), t.data_ptr() + nbytes) for t in w.kv_cache)
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:])), "layers overlap"
    p = [t.data_ptr() for t in w.kv_cache]
    assert p[3] - p[0] == nbytes and p[6] - p[3] == nbytes and p[4] - p[1] == nbytes     # stripe = layers l, l+3, l+6
    src_c = cpu_pool(L, NB, bs, H, D, torch.bfloat16, 51)
    for t, c in zip(w.kv_cache, src_c):
        t.copy_(c)
    si, di = [3, 4095, 0, 1717, 8], [1, 2, 3000, 31, 5]
    buf = w.extract_kv_blocks(si)
    assert same_bits(buf, orc.ref_extract_kv_blocks(src_c, si))
    w.write_kv_blocks(di, buf)
    orc.ref_write_kv_blocks(src_c, di, orc.ref_extract_kv_blocks(src_c, si))
    for l in range(L):
        assert same_bits(w.kv_cache[l], src_c[l]), f"layer {l}"
    # more stripes than layers, and no room for spacers
    layers = allocate_layers_spread(2, (2, 4, 16, 1, 8), torch.float16, torch.device(DEV), stripes=5,
                                    reserve_bytes=1 << 50)
    assert len(layers) == 2 and layers[0].data_ptr() != layers[1].data_ptr()
    kv_ops.kv_pack(PoolView(layers), [0, 3])
    torch.cuda.synchronize()
