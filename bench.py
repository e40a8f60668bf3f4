#!/usr/bin/env python3
"""Benchmark of the KV data-movement path on one MI355X.

Workload (default, ``qwen2_7b_migrate``): the Qwen2-7B KV shape — 28 layers of
``[2, 60000, 16, 4, 128]`` bf16 (51.3 GiB per pool) — and a batch of 32 migrating
requests with prompt lengths U{512..4096} plus a 1024-token image prefix
(96..320 blocks each). One *step* moves every request of the batch: pack from the
source pool under its block table into a contiguous transfer buffer
(``KVWorker.extract_kv_blocks``, one call per request as the reference does), then
unpack every buffer into a second, independently allocated pool under a different
table (``KVWorker.write_kv_blocks``, one call per request). Everything is resident in HBM before the timed
region (pools, block tables); values are synthetic N(0, 0.5).

Prints ONE JSON line. ``value`` is whole-job GB/s = algorithmic bytes (read +
write of pack and of unpack = 4 x payload) / wall time of the timed steps.
``roofline`` prices the block-move kernel (pack and unpack are two instances of
the same kernel) against the 8 TB/s HBM peak from HIP-event times of its launches
inside the timed region. ``cpu_baseline`` times the reference's torch expressions
(oracle ``ref_*``) on the host cores for a bounded sample of the same batch.
"""
import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--blocks", type=int, default=60000, help="pool size in blocks (the Qwen2-7B migration workload uses 60000)")
    ap.add_argument("--requests", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the secondary measurements (append, batched, copy)")
    ap.add_argument("--variant", type=int, default=0, help="block-move launch variant (tuning)")
    ap.add_argument("--spread", type=int, default=4,
                    help="stripes per pool: each pool's layers are allocated in this many pieces spread over the "
                         "free device memory (0 or 1: one allocation per pool)")
    ap.add_argument("--extended", action="store_true",
                    help="after the headline, free its pools and measure the fp8 70B-class shape and the ~200 GB "
                         "rebalancing shape at full size (adds about a minute)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 1 GiB copy with the same tile engine (a kernel of known traffic, "
                         "for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    return ap.parse_args()


def make_requests(num_requests, num_blocks, seed):
    """Block tables of the batch: disjoint slices of two different permutations."""
    g = torch.Generator().manual_seed(seed)
    prompts = torch.randint(512, 4097, (num_requests,), generator=g)
    nblk = [(int(p) + 1024 + 15) // 16 for p in prompts]
    total = sum(nblk)
    if total > num_blocks:
        raise SystemExit(f"pool of {num_blocks} blocks cannot hold the batch ({total} blocks)")
    sperm = torch.randperm(num_blocks, generator=g)
    dperm = torch.randperm(num_blocks, generator=torch.Generator().manual_seed(seed + 1000))
    tables, off = [], 0
    for n in nblk:
        tables.append((sperm[off:off + n].clone(), dperm[off:off + n].clone()))
        off += n
    return tables, total


def cpu_baseline(tables, L, bs, H, D, dtype, budget_s=15.0):
    """The reference's torch path on the host cores: the same batch (same block counts per
    request) on pools reduced to just hold it — bytes moved depend on the blocks per request,
    not on the pool size. Passes repeat until about `budget_s` seconds of CPU work are done."""
    from oracle import kv_oracle as orc

    nb = sum(len(s) for s, _ in tables)
    NBc = nb + 512
    torch.manual_seed(0)
    src = [torch.empty((2, NBc, bs, H, D), dtype=dtype).normal_(0.0, 0.5) for _ in range(L)]
    dst = [torch.zeros((2, NBc, bs, H, D), dtype=dtype) for _ in range(L)]
    g = torch.Generator().manual_seed(7)
    sp, dp = torch.randperm(NBc, generator=g), torch.randperm(NBc, generator=g)
    off, tabs = 0, []
    for s, _ in tables:
        tabs.append((sp[off:off + len(s)].tolist(), dp[off:off + len(s)].tolist()))
        off += len(s)
    chunk = bs * H * D * src[0].element_size()
    bytes_per_pass = 4 * nb * L * 2 * chunk
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 50):
        t0 = time.perf_counter()
        bufs = [orc.ref_extract_kv_blocks(src, si) for si, _ in tabs]
        for (_, di), buf in zip(tabs, bufs):
            orc.ref_write_kv_blocks(dst, di, buf)
        del bufs
        times.append(time.perf_counter() - t0)
    total = time.perf_counter() - t_start
    times.sort()
    med = times[len(times) // 2]
    return {
        "value": round(bytes_per_pass / med / 1e9, 3),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"the whole batch ({len(tabs)} requests, {nb} blocks, {bytes_per_pass / 1e9:.2f} GB algorithmic per "
                  f"pass) on host pools reduced to {NBc} blocks; the reference's torch indexing + stack / indexed "
                  f"assignment on CPU tensors; median of {len(times)} passes over {total:.1f} s ({med:.2f} s each)",
    }


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the cross-GPU hop is replaced by a second pool on the "
              "same device); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the KV kernels have no CPU fallback", file=sys.stderr)
        sys.exit(2)

    from elasticmm_amd import _lib, kv_ops
    from elasticmm_amd.kv_ops import PoolView
    from elasticmm_amd.worker import KVWorker

    if args.variant:
        # launch variants exist only in the hooks build of the library: route this process through it
        _lib.use_hooks_build().emm_hook_set_move_variant(args.variant)
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, bs, H, D, dtype = 28, 16, 4, 128, torch.bfloat16
    NB = args.blocks
    chunk = bs * H * D * 2
    tables, total_blocks = make_requests(args.requests, NB, seed=2)

    src_w, dst_w = KVWorker(0, "cuda:0", bs), KVWorker(1, "cuda:0", bs)
    src_w.init_kvcache(NB, num_layers=L, num_kv_heads=H, head_size=D, dtype=dtype, monolithic=True,
                       spread_stripes=args.spread)
    dst_w.init_kvcache(NB, num_layers=L, num_kv_heads=H, head_size=D, dtype=dtype, monolithic=True,
                       spread_stripes=args.spread)
    g = torch.Generator(device=dev).manual_seed(2)
    for t in src_w.kv_cache:
        t.normal_(0.0, 0.5, generator=g)
    for t in dst_w.kv_cache:
        t.zero_()
    dev_tables = [(s.to(dev), d.to(dev)) for s, d in tables]
    torch.cuda.synchronize()

    payload = total_blocks * L * 2 * chunk       # bytes held by the batch's blocks
    bytes_per_step = 4 * payload                 # pack: read + write, unpack: read + write

    def step(events=None):
        # pack every request on the source side, then unpack every request on the destination
        # side: 6 GB of transfer buffers lie between a buffer's pack and its unpack, so the
        # unpack reads come from HBM (not from the 256 MB Infinity Cache) as they would on a
        # receiving GPU.
        # HIP events bracket each phase (3 per step, on the launch stream), not each launch: an
        # event record between every two kernels costs several microseconds of idle GPU.
        if events is not None:
            e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
            e0.record()
        bufs = [src_w.extract_kv_blocks(si) for si, _ in dev_tables]
        if events is not None:
            e1.record()
        for k, (_, di) in enumerate(dev_tables):
            dst_w.write_kv_blocks(di, bufs[k])
        if events is not None:
            e2.record()
            events.append((e0, e1, e2))

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(events)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall = t1 - t0
    ms_per_step = wall / args.steps * 1e3
    value = bytes_per_step * args.steps / wall / 1e9

    # kernel time of the block-move kernel (pack and unpack instances) from the phase events:
    # each phase is 32 back-to-back launches of that kernel and nothing else
    pack_ms = sum(e0.elapsed_time(e1) for e0, e1, _ in events)
    unpack_ms = sum(e1.elapsed_time(e2) for _, e1, e2 in events)
    launches = 2 * len(dev_tables) * len(events)
    kern_bytes = 2 * 2 * payload * len(events)  # per step: pack 2 x payload + unpack 2 x payload
    achieved = kern_bytes / ((pack_ms + unpack_ms) * 1e-3) / 1e9
    roofline = {
        "bound": "hbm",
        "kernel": "emm_block_move_kernel (pack + unpack instances)",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBPS, 4),
        # HBM bytes per launch: rocprofv3 FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 (factors from a plain
        # 1 GiB copy in the same profile run) came to 1.0004 x the algorithmic bytes for this kernel on this
        # workload (profiles/block_move_qwen2_7b_migrate_pmc.txt); the figure is that ratio, not a live counter
        "traffic": int(kern_bytes / launches * 1.0004),
        "launches": launches,
        "avg_launch_us": round((pack_ms + unpack_ms) * 1e3 / launches, 2),
        "avg_bytes_per_launch": int(kern_bytes / launches),
        "pack_GBps": round(kern_bytes / 2 / (pack_ms * 1e-3) / 1e9, 1),
        "unpack_GBps": round(kern_bytes / 2 / (unpack_ms * 1e-3) / 1e9, 1),
    }

    if args.calibrate_copy:
        a = torch.empty(1 << 30, dtype=torch.uint8, device=dev).random_(0, 255)
        b = torch.empty_like(a)
        kv_ops.stream_copy(a, b)
        torch.cuda.synchronize()
        del a, b

    # spot check inside the bench: the last request really arrived
    si, di = dev_tables[-1]
    assert torch.equal(dst_w.kv_cache[L - 1][:, di], src_w.kv_cache[L - 1][:, si]), "migration check failed"

    extra = {}
    if not args.no_extra:
        extra = secondary(src_w, dst_w, dev_tables, payload, L, bs, H, D, NB, dev)

    if args.extended:
        src_w.kv_cache = dst_w.kv_cache = None
        src_w._pool = dst_w._pool = None
        dev_tables = None
        torch.cuda.empty_cache()
        extra["extended"] = extended(dev, args.spread)

    result = {
        "metric": "KV pack+unpack GB/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "u8",
        "data": "synthetic",
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "config": {
            "workload": "qwen2_7b_migrate: 28 layers x [2,%d,16,4,128] bf16 x 2 pools, %d requests (%d blocks, "
                        "%.2f GB payload), 32 per-request packs, then 32 per-request unpacks under different block tables"
                        % (NB, len(tables), total_blocks, payload / 1e9),
            "num_layers": L, "num_blocks": NB, "block_size": bs, "kv_heads": H, "head_dim": D,
            "requests": len(tables), "blocks_moved": total_blocks, "algorithmic_bytes_per_step": bytes_per_step,
            "pool_allocation": ("each pool allocated on its own, layers in %d stripes spread over the free device "
                                "memory" % args.spread) if args.spread > 1 else "each pool one allocation",
        },
        "roofline": roofline,
        "extra": extra,
    }
    if not args.no_cpu_baseline:
        # free the device pools first: the host leg needs nothing from them
        result["cpu_baseline"] = cpu_baseline(tables, L, bs, H, D, dtype)
    print(json.dumps(result), flush=True)


def _wall(fn):
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


def timed(fn, iters, warmup=2):
    """Median and min milliseconds of fn() over iters runs, HIP events on the current stream."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(iters):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        fn()
        e1.record()
        e1.synchronize()
        ts.append(e0.elapsed_time(e1))
    ts.sort()
    return ts[len(ts) // 2], ts[0]


def secondary(src_w, dst_w, dev_tables, payload, L, bs, H, D, NB, dev):
    """Other shapes of the same path, reported next to the headline (not bench lines of their own)."""
    from elasticmm_amd import cache_ops, kv_ops

    out = {}
    chunk = bs * H * D * 2
    sp, dp = src_w.pool, dst_w.pool
    # one launch for the whole batch (concatenated tables)
    all_si = torch.cat([s for s, _ in dev_tables])
    all_di = torch.cat([d for _, d in dev_tables])
    buf = torch.empty(sp.packed_shape(all_si.numel()), dtype=sp.dtype, device=dev)
    med, mn = timed(lambda: kv_ops.kv_pack(sp, all_si, out=buf), 10)
    out["batched_pack_GBps"] = round(2 * payload / (med * 1e-3) / 1e9, 1)
    med, mn = timed(lambda: kv_ops.kv_unpack(dp, all_di, buf), 10)
    out["batched_unpack_GBps"] = round(2 * payload / (med * 1e-3) / 1e9, 1)
    med, mn = timed(lambda: kv_ops.kv_migrate(sp, all_si, dp, all_di), 10)
    out["fused_migrate_GBps"] = round(2 * payload / (med * 1e-3) / 1e9, 1)
    def interleaved():
        for si, di in dev_tables:
            dst_w.write_kv_blocks(di, src_w.extract_kv_blocks(si))

    med, mn = timed(interleaved, 5)
    out["per_request_pack_then_unpack_interleaved_GBps"] = round(4 * payload / (med * 1e-3) / 1e9, 1)
    # yardsticks: plain copies of the same byte count
    flat = buf.view(-1)
    other = torch.empty_like(flat)
    med, mn = timed(lambda: kv_ops.stream_copy(flat, other), 10)
    out["plain_copy_same_engine_GBps"] = round(2 * payload / (med * 1e-3) / 1e9, 1)
    med, mn = timed(lambda: other.copy_(flat), 10)
    out["torch_copy_GBps"] = round(2 * payload / (med * 1e-3) / 1e9, 1)
    del other, buf
    # copy_blocks: half of the batch's blocks to free blocks of the same pool
    P = all_si.numel() // 2
    used = torch.zeros(NB, dtype=torch.bool, device=dev)
    used[all_si] = True
    free = (~used).nonzero().squeeze(1)
    if free.numel() >= P:
        mapping = torch.stack([all_si[:P], free[:P]], 1).contiguous()
        med, mn = timed(lambda: kv_ops.copy_blocks(sp, mapping), 10)
        out["copy_blocks_GBps"] = round(2 * P * L * 2 * chunk / (med * 1e-3) / 1e9, 1)
    out["append"] = append_bench(src_w.kv_cache, NB, bs, H, D, torch.bfloat16, None, None, dev)
    out["append_paged_layout"] = paged_append_bench(src_w.kv_cache, NB, bs, H, D, dev)
    return out


def paged_append_bench(kv, NB, bs, H, D, dev, T=8448, decode=256):
    """The same step appended into the paged-attention layout (key [NB,H,D/8,bs,8], value [NB,H,D,bs],
    viewed over the same pool memory): `decode` single tokens in random blocks, then one prompt of
    T - decode tokens that fills blocks in order (its blocks start off the 16-token grid of the token
    list). Bytes: 2 x 2 x row per token, as for the flash layout."""
    from elasticmm_amd import cache_ops

    L = len(kv)
    x = 16 // kv[0].element_size()
    g = torch.Generator(device=dev).manual_seed(4)
    blocks = torch.randperm(NB, device=dev, generator=g)
    dec = blocks[:decode] * bs + torch.randint(bs, (decode,), device=dev, generator=g)
    nb_prompt = (T - decode + bs - 1) // bs + 1
    prompt = (blocks[decode:decode + nb_prompt, None] * bs + torch.arange(bs, device=dev)[None, :]).reshape(-1)
    first = bs - 5  # the prompt resumes 5 slots before a block boundary
    slots = torch.cat([dec, prompt[first:first + T - decode]]).contiguous()
    keys = [torch.randn((T, H, D), device=dev, generator=g).to(torch.bfloat16) for _ in range(L)]
    values = [torch.randn((T, H, D), device=dev, generator=g).to(torch.bfloat16) for _ in range(L)]
    kcs = [kv[l][0].view(NB, H, D // x, bs, x) for l in range(L)]
    vcs = [kv[l][1].view(NB, H, D, bs) for l in range(L)]
    step_bytes = L * (T * 2 * H * D * 2 * 2 + 8 * T)

    def per_layer():
        for l in range(L):
            cache_ops.reshape_and_cache(keys[l], values[l], kcs[l], vcs[l], slots, "auto")

    def entry(ms):
        return {"tokens_per_s": round(T / (ms * 1e-3)), "ms_per_step": round(ms, 4),
                "GBps": round(step_bytes / (ms * 1e-3) / 1e9, 1)}

    res = {"T": T, "decode_tokens": decode, "layers": L, "algorithmic_bytes_per_step": step_bytes}
    med, _ = timed(per_layer, 20)
    res["per_layer_calls_eager"] = entry(med)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        per_layer()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        per_layer()
    med, _ = timed(graph.replay, 20)
    res["per_layer_calls_hip_graph"] = entry(med)
    plan = cache_ops.paged_layered_append(keys, values, kcs, vcs)
    med, _ = timed(lambda: plan(slots), 20)
    res["one_launch_all_layers"] = entry(med)
    # a decode-only step: every token alone in its block (each 2-byte V element and each 16-byte K piece
    # lands in a cache line of its own, so the memory system rewrites the token's whole block region)
    Td = 256
    dplan = cache_ops.paged_layered_append([k[:Td] for k in keys], [v[:Td] for v in values], kcs, vcs)
    dslots = dec[:Td].contiguous() if decode >= Td else slots[:Td].contiguous()
    med, _ = timed(lambda: dplan(dslots), 20)
    res["decode_only_256_tokens_one_launch"] = {"tokens_per_s": round(Td / (med * 1e-3)), "ms_per_step": round(med, 4),
                                                "GBps": round(L * Td * 2 * H * D * 4 / (med * 1e-3) / 1e9, 1)}
    return res


def append_bench(kv, NB, bs, H, D, cache_dtype_name, k_scales, v_scales, dev, T=8448):
    """reshape_and_cache for one step: 256 decode tokens + one 8192-token prefill chunk, slots random
    over the pool, 5 % padded (-1). Three ways of issuing it: the vLLM-shaped call once per layer
    (eager Python), the same L launches replayed from a HIP graph, and one launch for all layers from
    a prepared plan. tokens/s = valid tokens / time of all layers."""
    from elasticmm_amd import cache_ops

    L = len(kv)
    fp8 = kv[0].element_size() == 1
    mode = "fp8" if fp8 else "auto"
    g = torch.Generator(device=dev).manual_seed(3)
    slots = torch.randperm(NB * bs, device=dev, generator=g)[:T].clone()
    slots[torch.rand(T, device=dev, generator=g) < 0.05] = -1
    valid = int((slots >= 0).sum())
    keys = [torch.randn((T, H, D), device=dev, generator=g).to(torch.bfloat16) for _ in range(L)]
    values = [torch.randn((T, H, D), device=dev, generator=g).to(torch.bfloat16) for _ in range(L)]
    row = H * D
    step_bytes = L * (valid * 2 * row * (2 + kv[0].element_size()) + 8 * T)
    ks = [None] * L if not fp8 else [k_scales[l:l + 1] for l in range(L)]
    vs = [None] * L if not fp8 else [v_scales[l:l + 1] for l in range(L)]

    def per_layer():
        for l in range(L):
            cache_ops.reshape_and_cache_flash(keys[l], values[l], kv[l][0], kv[l][1], slots, mode, ks[l], vs[l])

    def entry(ms):
        return {"tokens_per_s": round(valid / (ms * 1e-3)), "ms_per_step": round(ms, 4),
                "GBps": round(step_bytes / (ms * 1e-3) / 1e9, 1)}

    res = {"T": T, "valid": valid, "layers": L, "algorithmic_bytes_per_step": step_bytes}
    med, _ = timed(per_layer, 20)
    res["per_layer_calls_eager"] = entry(med)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        per_layer()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        per_layer()
    med, _ = timed(graph.replay, 20)
    res["per_layer_calls_hip_graph"] = entry(med)
    plan = cache_ops.layered_append(keys, values, kv, mode, k_scales, v_scales)
    med, _ = timed(lambda: plan(slots), 20)
    res["one_launch_all_layers"] = entry(med)
    return res


def extended(dev, spread=4):
    """The two other target shapes at full size (run with --extended; needs the whole GPU):
    the fp8-e4m3 70B-class per-GPU shape and the elastic rebalancing of a ~200 GB pool."""
    from elasticmm_amd import kv_ops
    from elasticmm_amd.kv_ops import PoolView

    out = {}
    # ---- fp8: 80 layers x [2, NB, 16, 8, 128] e4m3, 64 requests of U{1024..8192} tokens
    L, bs, H, D, NB = 80, 16, 8, 128, 20000
    chunk = bs * H * D
    g = torch.Generator().manual_seed(4)
    lens = torch.randint(1024, 8193, (64,), generator=g)
    nblk = [(int(t) + 15) // 16 for t in lens]
    total = sum(nblk)
    perm_s = torch.randperm(NB, generator=g)[:total].to(dev)
    perm_d = torch.randperm(NB, generator=g)[:total].to(dev)
    k_scales = (torch.rand(L, generator=g) * 0.09 + 0.01).to(dev)
    v_scales = (torch.rand(L, generator=g) * 0.09 + 0.01).to(dev)
    from elasticmm_amd.worker import allocate_layers_spread

    def make_pool(dtype):
        shape = (2, NB, bs, H, D)
        if spread > 1:
            return allocate_layers_spread(L, shape, dtype, dev, spread)
        return list(torch.empty((L,) + shape, dtype=dtype, device=dev).unbind(0))

    src = make_pool(torch.uint8)
    dst = make_pool(torch.uint8)
    for t in src:
        t.random_(0, 0x78)  # finite positive e4m3 bytes
    for t in dst:
        t.zero_()
    sp, dp = PoolView(src), PoolView(dst)
    off, ts_pack, ts_unpack, payload = 0, 0.0, 0.0, 0
    for n in nblk:  # per-request staging buffers (the whole batch would be 45 GiB)
        si, di = perm_s[off:off + n], perm_d[off:off + n]
        buf = torch.empty(sp.packed_shape(n), dtype=torch.uint8, device=dev)
        med, _ = timed(lambda: kv_ops.kv_pack(sp, si, out=buf), 3, warmup=1)
        ts_pack += med
        med, _ = timed(lambda: kv_ops.kv_unpack(dp, di, buf), 3, warmup=1)
        ts_unpack += med
        payload += n * L * 2 * chunk
        off += n
        del buf
    out["fp8_70b_shape"] = {"layers": L, "pool_blocks": NB, "requests": 64, "blocks": total,
                            "payload_GB": round(payload / 1e9, 2),
                            "pack_GBps": round(2 * payload / (ts_pack * 1e-3) / 1e9, 1),
                            "unpack_GBps": round(2 * payload / (ts_unpack * 1e-3) / 1e9, 1)}
    out["fp8_70b_shape"]["append"] = append_bench(src, NB, bs, H, D, "fp8", k_scales, v_scales, dev)
    del dst, dp
    torch.cuda.empty_cache()
    # dequantising unpack into a bf16 pool (first 16 requests)
    dq = make_pool(torch.bfloat16)
    for t in dq:
        t.zero_()
    dqp = PoolView(dq)
    off, t_dq, pay = 0, 0.0, 0
    for n in nblk[:16]:
        buf = kv_ops.kv_pack(sp, perm_s[off:off + n])
        di = perm_d[off:off + n]
        med, _ = timed(lambda: kv_ops.kv_unpack_dequant_fp8(dqp, di, buf, k_scales, v_scales), 3, warmup=1)
        t_dq += med
        pay += n * L * 2 * chunk
        off += n
        del buf
    out["fp8_70b_shape"]["dequant_unpack_GBps"] = round(3 * pay / (t_dq * 1e-3) / 1e9, 1)
    del src, sp, dq, dqp
    torch.cuda.empty_cache()

    # ---- GPU <-> CPU swap (pinned host pool, kernels read / write it over PCIe): Qwen2-7B layout
    from elasticmm_amd.worker import KVWorker
    w = KVWorker(0, "cuda:0", 16)
    w.init_kvcache(4096, 2048, num_layers=28, num_kv_heads=4, head_size=128, dtype=torch.bfloat16)
    for t in w.kv_cache:
        t.normal_(0.0, 0.5)
    gsw = torch.Generator().manual_seed(6)
    nsw = 1024
    gpu_ids = torch.randperm(4096, generator=gsw)[:nsw].to(dev)
    cpu_ids = torch.randperm(2048, generator=gsw)[:nsw].to(dev)
    sw_bytes = nsw * 28 * 2 * 16 * 4 * 128 * 2

    def swap(is_in):
        w.swap_blocks(["r"], cpu_ids if is_in else gpu_ids, gpu_ids if is_in else cpu_ids, is_in)
        (w.swap_in_stream if is_in else w.swap_out_stream).synchronize()

    t_out = min(_wall(lambda: swap(False)) for _ in range(4))
    t_in = min(_wall(lambda: swap(True)) for _ in range(4))
    stage_g = torch.empty(sw_bytes, dtype=torch.uint8, device=dev)
    stage_c = torch.empty(sw_bytes, dtype=torch.uint8, pin_memory=True)

    def d2h():
        stage_c.copy_(stage_g, non_blocking=True)
        torch.cuda.synchronize()

    def h2d():
        stage_g.copy_(stage_c, non_blocking=True)
        torch.cuda.synchronize()

    t_d2h = min(_wall(d2h) for _ in range(4))
    t_h2d = min(_wall(h2d) for _ in range(4))
    out["swap_pcie"] = {"blocks": nsw, "GB": round(sw_bytes / 1e9, 3),
                        "swap_out_GBps": round(sw_bytes / t_out / 1e9, 1), "swap_in_GBps": round(sw_bytes / t_in / 1e9, 1),
                        "contiguous_memcpy_d2h_GBps": round(sw_bytes / t_d2h / 1e9, 1),
                        "contiguous_memcpy_h2d_GBps": round(sw_bytes / t_h2d / 1e9, 1)}
    del w, stage_g, stage_c
    torch.cuda.empty_cache()

    # ---- rebalancing: ~200 GB bf16 pool in the Qwen2-7B layout, move 50 % of the live half
    L, bs, H, D = 28, 16, 4, 128
    chunk = bs * H * D * 2
    NB = 218000
    pool = torch.empty((L, 2, NB, bs, H, D), dtype=torch.bfloat16, device=dev)
    for l in range(L):
        pool[l].normal_(0.0, 0.5)
    pv = PoolView(pool)
    g = torch.Generator().manual_seed(5)
    perm = torch.randperm(NB, generator=g)
    live = perm[:NB // 2]
    free = perm[NB // 2:]
    P = live.numel() // 2
    mapping = torch.stack([live[:P], free[:P]], 1).contiguous().to(dev)
    med, mn = timed(lambda: kv_ops.copy_blocks(pv, mapping), 5, warmup=1)
    ok = bool(torch.equal(pool[3][:, mapping[:1000, 1]], pool[3][:, mapping[:1000, 0]]))
    out["rebalance_200GB"] = {"pool_GB": round(pool.numel() * 2 / 1e9, 1), "pairs": P,
                              "algorithmic_GB": round(2 * P * L * 2 * chunk / 1e9, 1), "ms": round(med, 3),
                              "copy_blocks_GBps": round(2 * P * L * 2 * chunk / (med * 1e-3) / 1e9, 1),
                              "spot_check": ok}
    # vision-embedding gather interleaved on the same stream
    imgs = torch.randint(64, 2305, (128,), generator=g).tolist()
    embeds = [torch.randn((p_, 3584), device=dev).to(torch.bfloat16) for p_ in imgs]
    vis_bytes = 2 * sum(imgs) * 3584 * 2
    outbuf = torch.empty((sum(imgs), 3584), dtype=torch.bfloat16, device=dev)
    med, _ = timed(lambda: kv_ops.concat_rows(embeds, out=outbuf), 10)
    out["rebalance_200GB"]["vision_concat"] = {"images": 128, "rows": sum(imgs), "ms": round(med, 4),
                                               "GBps": round(vis_bytes / (med * 1e-3) / 1e9, 1)}
    # the same gather from segments prepared when the embeddings entered the cache (what
    # KVWorker.gather_vision_embeddings does): the host reads two fields per image instead of the tensors
    prepared = [kv_ops.RowSource(e) for e in embeds]
    med, _ = timed(lambda: kv_ops.concat_row_sources(prepared, out=outbuf), 10)
    out["rebalance_200GB"]["vision_concat"]["prepared_segments_ms"] = round(med, 4)
    out["rebalance_200GB"]["vision_concat"]["prepared_segments_GBps"] = round(vis_bytes / (med * 1e-3) / 1e9, 1)
    med_t, _ = timed(lambda: torch.cat(embeds, 0, out=outbuf), 10)
    out["rebalance_200GB"]["vision_concat"]["torch_cat_GBps"] = round(vis_bytes / (med_t * 1e-3) / 1e9, 1)
    quarter = mapping[:P // 8]

    def interleaved():
        for k in range(8):
            kv_ops.copy_blocks(pv, mapping[k * (P // 8):(k + 1) * (P // 8)])
            kv_ops.concat_rows(embeds[k * 16:(k + 1) * 16], out=outbuf[:sum(imgs[k * 16:(k + 1) * 16])])

    med, _ = timed(interleaved, 3, warmup=1)
    tot = 2 * (P // 8) * 8 * L * 2 * chunk + vis_bytes
    out["rebalance_200GB"]["interleaved_copy_and_concat_GBps"] = round(tot / (med * 1e-3) / 1e9, 1)
    del quarter
    return out


if __name__ == "__main__":
    main()
