#!/usr/bin/env python3
"""Benchmark of the KV data-movement path on one MI355X.

Headline workload (``qwen2_7b_migrate``): the Qwen2-7B KV shape — 28 layers of
``[2, 60000, 16, 4, 128]`` bf16 (51.3 GiB per pool) — and a batch of 32 migrating
requests with prompt lengths U{512..4096} plus a 1024-token image prefix
(96..320 blocks each). One *step* moves every request of the batch: pack from the
source pool under its block table into a contiguous transfer buffer
(``KVWorker.extract_kv_blocks``, one call per request as the reference does), then
unpack every buffer into a second, independently allocated pool under a different
table (``KVWorker.write_kv_blocks``, one call per request). Everything is resident in
HBM before the timed region (pools, block tables); values are synthetic N(0, 0.5).

Prints ONE JSON line. ``value`` is whole-job GB/s = algorithmic bytes (read + write of
pack and of unpack = 4 x payload) / wall time of the timed steps. ``roofline`` prices the
block-move kernel (pack and unpack are two instances of the same kernel) against the
8 TB/s HBM peak from HIP-event times of its launches inside the timed region.
``cpu_baseline`` times the reference's torch expressions (oracle ``ref_*``) on the host
cores for bounded samples of the same workloads.

``extra`` holds the other shapes of the path, each with its own algorithmic bytes, rate,
fraction of the 8 TB/s peak, kernel name and average launch time:
  allocation_modes   the headline again with each pool in one allocation and with one
                     allocation per layer (what a pool adopted from vLLM looks like); probes of
                     what the scalar fetches in front of a pack's loads cost
  list_indices       the headline with block tables passed as Python lists (the reference's
                     call shape; the ids travel in the kernel argument block)
  batched / fused    one launch for the whole batch; fused pool-to-pool migrate; copy_blocks;
                     the per-request launches alternating over two streams against one
  ceilings           what this memory system does for the same access patterns without the
                     other half of the copy (sequential / gathered reads, sequential /
                     scattered writes, plain copy), from the hooks build of the library
  append             reshape_and_cache for one step (config 3): per-layer calls eager / from a
                     HIP graph, one launch for all layers, a 256-token decode step, and the
                     launch-bound yardsticks (plain copy of the same bytes, empty launch)
  append_paged_layout, cfg1_latency, fp8_70b_shape (config 4), rebalance_200GB (config 5,
  with the vision gather on the same and on a second stream), swap_pcie
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
ALL_SECTIONS = ["batched", "ceilings", "append", "paged", "lists", "modes", "cfg1", "fp8", "rebalance", "swap", "variants", "placement"]


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--blocks", type=int, default=60000, help="pool size in blocks (the Qwen2-7B migration workload uses 60000)")
    ap.add_argument("--requests", type=int, default=32)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="headline only (same as --sections none)")
    ap.add_argument("--sections", default="all",
                    help="comma-separated secondary measurements to run: " + ",".join(ALL_SECTIONS) + " (all | none)")
    ap.add_argument("--variant", type=lambda v: int(v, 0), default=0,
                    help="launch variant of the hooks build (tuning; routes every call through libemm_kv_hooks.so)")
    ap.add_argument("--spread", type=int, default=0,
                    help="stripes per pool of the headline: k > 1 allocates each pool's layers in k pieces spread over the "
                         "free device memory (KVWorker.init_kvcache(spread_stripes=k)); 0 (default): the reference's own "
                         "layout, one torch.empty per layer (what bind_kv_cache adopts from vLLM)")
    ap.add_argument("--weights-gib", type=float, default=-1.0,
                    help="size of the allocation made before the pools, standing for the model's weights, which a "
                         "serving worker loads before it sizes and allocates its KV pool (default: the weights of the "
                         "configuration's model; 0 = allocate the pools first)")
    ap.add_argument("--monolithic", action="store_true",
                    help="with --spread 0: one allocation per pool (init_kvcache's default) instead of one per layer")
    ap.add_argument("--no-append-context", action="store_true",
                    help="skip extra.append.in_context (HIP graphs that fork over several streams or contain library GEMMs; "
                         "rocprofv3 --pmc has crashed replaying them)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch one plain 1 GiB copy with the same tile engine (a kernel of known traffic, "
                         "for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    return ap.parse_args()


# ---------------------------------------------------------------------------------------------- helpers
def rec(nbytes, ms, launches=1, kernel=None, **more):
    """One measurement: algorithmic bytes, milliseconds, rate, fraction of the HBM peak."""
    gbps = nbytes / (ms * 1e-3) / 1e9
    out = {"GBps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4), "ms": round(ms, 4),
           "algorithmic_bytes": int(nbytes), "launches": launches,
           "avg_launch_us": round(ms * 1e3 / launches, 2)}
    if kernel:
        out["kernel"] = kernel
    out.update(more)
    return out


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


def _wall(fn):
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


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


def measure_migrate(src_w, dst_w, tabs, steps, warmup, payload):
    """`steps` timed steps of: pack every request on the source side, then unpack every request on the
    destination side. All packs run before the unpacks: 6 GB of transfer buffers lie between a buffer's
    pack and its unpack, so the unpack reads come from HBM (not from the 256 MB Infinity Cache) as they
    would on a receiving GPU. HIP events bracket each phase (3 per step, on the launch stream), not each
    launch: an event record between every two kernels costs several microseconds of idle GPU."""
    def step(events=None):
        if events is not None:
            e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
            e0.record()
        bufs = [src_w.extract_kv_blocks(si) for si, _ in tabs]
        if events is not None:
            e1.record()
        for k, (_, di) in enumerate(tabs):
            dst_w.write_kv_blocks(di, bufs[k])
        if events is not None:
            e2.record()
            events.append((e0, e1, e2))

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    events = []
    t0 = time.perf_counter()
    for _ in range(steps):
        step(events)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    pack_ms = sum(e0.elapsed_time(e1) for e0, e1, _ in events)
    unpack_ms = sum(e1.elapsed_time(e2) for _, e1, e2 in events)
    launches = 2 * len(tabs) * steps
    kern_bytes = 4 * payload * steps
    return {
        "value": 4 * payload * steps / wall / 1e9,
        "ms_per_step": wall / steps * 1e3,
        "kernel_GBps": kern_bytes / ((pack_ms + unpack_ms) * 1e-3) / 1e9,
        "pack_GBps": kern_bytes / 2 / (pack_ms * 1e-3) / 1e9,
        "unpack_GBps": kern_bytes / 2 / (unpack_ms * 1e-3) / 1e9,
        "launches": launches,
        "avg_launch_us": (pack_ms + unpack_ms) * 1e3 / launches,
        "avg_bytes_per_launch": kern_bytes / launches,
    }


def make_workers(NB, L, bs, H, D, dtype, dev, spread, monolithic=True, fill=True):
    from elasticmm_amd.worker import KVWorker

    src_w, dst_w = KVWorker(0, "cuda:0", bs), KVWorker(1, "cuda:0", bs)
    for w in (src_w, dst_w):
        w.init_kvcache(NB, num_layers=L, num_kv_heads=H, head_size=D, dtype=dtype, monolithic=monolithic,
                       spread_stripes=spread)
    if fill:
        g = torch.Generator(device=dev).manual_seed(2)
        for t in src_w.kv_cache:
            t.normal_(0.0, 0.5, generator=g)
    for t in dst_w.kv_cache:
        t.zero_()
    torch.cuda.synchronize()
    return src_w, dst_w


def release(*workers):
    for w in workers:
        w.kv_cache = None
        w._pool = None
    torch.cuda.empty_cache()


# Bytes of the models' weights. A worker of the reference loads the model (elasticmm/engine/v0/worker.py:256), measures
# what is left (:271-356) and only then allocates the KV pool (:358-394), so a pool never lies where a fresh process's
# first allocations land. Where the pools land matters for scattered writes on this part (bench `extra.placement`).
QWEN2_7B_WEIGHT_BYTES = 7_615_616_512 * 2   # bf16
LLAMA_70B_FP8_WEIGHT_BYTES = 70_553_706_496  # 70B-class, fp8 weights beside the fp8 KV cache


def weights_placeholder(args, nbytes, dev):
    """One allocation of the model's weight bytes (or of --weights-gib), made before the pools and kept alive while
    they are measured. Returns (tensor or None, GiB)."""
    if args.weights_gib >= 0:
        nbytes = int(args.weights_gib * (1 << 30))
    if nbytes <= 0:
        return None, 0.0
    w = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    w.zero_()
    return w, round(nbytes / (1 << 30), 3)


# ---------------------------------------------------------------------------------------------- CPU baselines
def host_cpu():
    """Threads for the CPU legs and what the host is: every core this process may use — os.cpu_count(), capped by
    OMP_NUM_THREADS where the environment sets it (a GPU box gives each job a share of its cores)."""
    n = os.cpu_count() or 1
    try:
        n = min(n, len(os.sched_getaffinity(0)))
    except (AttributeError, OSError):
        pass
    cap = os.environ.get("OMP_NUM_THREADS", "")
    if cap.isdigit() and int(cap) > 0:
        n = min(n, int(cap))
    torch.set_num_threads(n)
    model = "unknown"
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    return {"cores": torch.get_num_threads(), "os_cpu_count": os.cpu_count(), "cpu_model": model}


def cpu_baseline(tables, L, bs, H, D, dtype, budget_s=8.0):
    """The reference's torch path on the host cores: the same batch (same block counts per
    request) on pools reduced to just hold it — bytes moved depend on the blocks per request,
    not on the pool size. Passes repeat until about `budget_s` seconds of CPU work are done."""
    from oracle import kv_oracle as orc

    host_cpu()  # sets the thread count before anything is timed
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
        **host_cpu(),
        "kind": "port",
        "sample": f"the whole batch ({len(tabs)} requests, {nb} blocks, {bytes_per_pass / 1e9:.2f} GB algorithmic per "
                  f"pass) on host pools reduced to {NBc} blocks; the reference's torch indexing + stack / indexed "
                  f"assignment on CPU tensors; median of {len(times)} passes over {total:.1f} s ({med:.2f} s each)",
    }


def cpu_baseline_append(budget_s=5.0, L=28, bs=16, H=4, D=128, T=8448):
    """Config 3 on the host: the closed form of reshape_and_cache_flash (index_copy_ of the valid rows) per
    layer, same T, same 5 % padded slots, pool reduced to 2048 blocks (bytes moved depend on T, not on the pool)."""
    from oracle import kv_oracle as orc

    host_cpu()
    NBc = 2048
    g = torch.Generator().manual_seed(3)
    slots = torch.randperm(NBc * bs, generator=g)[:T].clone()
    slots[torch.rand(T, generator=g) < 0.05] = -1
    valid = int((slots >= 0).sum())
    key = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    value = torch.randn((T, H, D), generator=g).to(torch.bfloat16)
    caches = [torch.zeros((2, NBc, bs, H, D), dtype=torch.bfloat16) for _ in range(L)]
    step_bytes = L * (valid * 2 * H * D * 4 + 8 * T)
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < 200):
        t0 = time.perf_counter()
        for l in range(L):
            orc.ref_reshape_and_cache_flash(key, value, caches[l][0], caches[l][1], slots)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(valid / med), "unit": "tokens/s", "GBps": round(step_bytes / med / 1e9, 2),
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"one step of {T} tokens ({valid} valid) x {L} layers, per-layer index_copy_ of the valid rows on "
                      f"CPU tensors, pool reduced to {NBc} blocks; median of {len(times)} steps ({med * 1e3:.1f} ms each)"}


def cpu_baseline_cfg1(budget_s=2.0):
    """Config 1 exactly as specified, on the host."""
    from oracle import kv_oracle as orc

    host_cpu()
    L, NB, bs, H, D = 4, 1024, 16, 8, 128
    g = torch.Generator().manual_seed(0)
    src = [torch.randn((2, NB, bs, H, D), generator=g).to(torch.float16) for _ in range(L)]
    dst = [torch.zeros((2, NB, bs, H, D), dtype=torch.float16) for _ in range(L)]
    si = torch.randperm(NB, generator=g)[:32].tolist()
    di = torch.randperm(NB, generator=torch.Generator().manual_seed(1))[:32].tolist()
    nbytes = 4 * 32 * L * 2 * bs * H * D * 2
    times = []
    t_start = time.perf_counter()
    while len(times) < 5 or (time.perf_counter() - t_start < budget_s and len(times) < 2000):
        t0 = time.perf_counter()
        orc.ref_write_kv_blocks(dst, di, orc.ref_extract_kv_blocks(src, si))
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "us_per_pack_plus_unpack": round(med * 1e6, 1),
            "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"config 1 (4 layers x [2,1024,16,8,128] fp16, one request of 32 blocks), extract + write on "
                      f"CPU tensors; median of {len(times)} passes"}


def layout_name(args):
    if args.spread > 1:
        return "pools allocated with init_kvcache(spread_stripes=%d)" % args.spread
    if args.monolithic:
        return "one allocation per pool (init_kvcache's default)"
    return ("the reference's pool layout: one torch.empty per layer and pool, as vLLM's CacheEngine allocates and "
            "bind_kv_cache adopts (elasticmm/engine/v0/worker.py:388-394)")


# ---------------------------------------------------------------------------------------------- main
def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the cross-GPU hop is replaced by a second pool on the "
              "same device); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the KV kernels have no CPU fallback", file=sys.stderr)
        sys.exit(2)
    if args.no_extra or args.sections == "none":
        sections = set()
    elif args.sections == "all":
        sections = set(ALL_SECTIONS)
    else:
        sections = set(args.sections.split(","))
        unknown = sections - set(ALL_SECTIONS)
        if unknown:
            raise SystemExit(f"unknown sections: {sorted(unknown)}")

    from elasticmm_amd import _lib, kv_ops

    global APPEND_CONTEXT
    APPEND_CONTEXT = not args.no_append_context
    if args.variant:
        # launch variants exist only in the hooks build of the library: route this process through it
        _lib.use_hooks_build().emm_hook_set_move_variant(args.variant)
    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    L, bs, H, D, dtype = 28, 16, 4, 128, torch.bfloat16
    NB = args.blocks
    chunk = bs * H * D * 2
    tables, total_blocks = make_requests(args.requests, NB, seed=2)
    payload = total_blocks * L * 2 * chunk       # bytes held by the batch's blocks
    bytes_per_step = 4 * payload                 # pack: read + write, unpack: read + write

    # The headline runs on the reference's own pool layout: one torch.empty per layer (the list bind_kv_cache adopts
    # from vLLM's CacheEngine, elasticmm/engine/v0/worker.py:388-394). Other layouts: --spread / --monolithic, and
    # extra.allocation_modes.
    weights, weights_gib = weights_placeholder(args, QWEN2_7B_WEIGHT_BYTES, dev)
    src_w, dst_w = make_workers(NB, L, bs, H, D, dtype, dev, args.spread, monolithic=args.monolithic)
    dev_tables = [(s.to(dev), d.to(dev)) for s, d in tables]
    torch.cuda.synchronize()

    m = measure_migrate(src_w, dst_w, dev_tables, args.steps, args.warmup, payload)
    # HBM bytes per launch from rocprofv3: FETCH_SIZE x 2.000 + WRITE_SIZE x 1.000 (factors from a plain 1 GiB
    # copy in the same profile run) came to TRAFFIC_RATIO x the algorithmic bytes for this kernel on this
    # workload (profiles/block_move_qwen2_7b_migrate_pmc.txt). A counter cannot be read inside this process;
    # the figure below is that constant applied to this run's bytes per launch, not a reading of this run.
    TRAFFIC_RATIO = 1.0005
    roofline = {
        "bound": "hbm",
        "kernel": "emm_block_move_kernel (pack + unpack instances)",
        "achieved": round(m["kernel_GBps"], 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(m["kernel_GBps"] / HBM_PEAK_GBPS, 4),
        "traffic": int(m["avg_bytes_per_launch"] * TRAFFIC_RATIO),
        "traffic_source": "a constant, not a counter read in this run: %.4f x this run's algorithmic bytes per launch. The "
                          "ratio is rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE per dispatch of this kernel on this workload, "
                          "scaled by a plain copy of known size, as recorded in profiles/block_move_qwen2_7b_migrate_pmc.txt "
                          "(regenerated whenever the kernel changes; the file states its command)" % TRAFFIC_RATIO,
        "launches": m["launches"],
        "avg_launch_us": round(m["avg_launch_us"], 2),
        "avg_bytes_per_launch": int(m["avg_bytes_per_launch"]),
        "pack_GBps": round(m["pack_GBps"], 1),
        "unpack_GBps": round(m["unpack_GBps"], 1),
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
    if "lists" in sections:
        list_tables = [(s.tolist(), d.tolist()) for s, d in tables]
        ml = measure_migrate(src_w, dst_w, list_tables, max(3, args.steps // 4), 1, payload)
        extra["list_indices"] = {
            "what": "the headline with block tables passed as Python lists (the reference's call shape): every call "
                    "checks the ids on the host, stages them in pinned memory and copies them to the device",
            "value_GBps": round(ml["value"], 1), "frac": round(ml["value"] / HBM_PEAK_GBPS, 4),
            "ms_per_step": round(ml["ms_per_step"], 4), "pack_GBps": round(ml["pack_GBps"], 1),
            "unpack_GBps": round(ml["unpack_GBps"], 1)}
    if "batched" in sections:
        extra.update(batched(src_w, dst_w, dev_tables, payload, L, chunk, NB, dev))
    if "ceilings" in sections:
        extra["ceilings"] = ceilings(src_w, dst_w, dev_tables, payload, dev)
    if "variants" in sections:
        extra["pack_variants"] = pack_variants(src_w, dev_tables, payload, dev)
    if "append" in sections:
        extra["append"] = append_bench(src_w.kv_cache, NB, bs, H, D, None, None, dev)
    if "paged" in sections:
        extra["append_paged_layout"] = paged_append_bench(src_w.kv_cache, NB, bs, H, D, dev)
    if "placement" in sections:
        extra["placement"] = placement(src_w, dst_w, dev_tables, payload, dev)
    release(src_w, dst_w)
    dev_tables = None
    if "placement" in sections:
        # with the weights' allocation still in place: the same pools freed and allocated again
        extra["placement"]["headline_on_pools_freed_and_allocated_again"] = reallocation_cycles(
            args, tables, NB, L, bs, H, D, dtype, payload, dev)

    if "modes" in sections:
        modes = {}
        for name, spread, mono in (("one_allocation_per_pool", 0, True), ("four_stripes_per_pool", 4, False)):
            sw, dw = make_workers(NB, L, bs, H, D, dtype, dev, spread, monolithic=mono)
            tabs = [(s.to(dev), d.to(dev)) for s, d in tables]
            mm = measure_migrate(sw, dw, tabs, max(3, args.steps // 4), 2, payload)
            modes[name] = {"value_GBps": round(mm["value"], 1), "frac": round(mm["value"] / HBM_PEAK_GBPS, 4),
                           "pack_GBps": round(mm["pack_GBps"], 1), "unpack_GBps": round(mm["unpack_GBps"], 1),
                           "avg_launch_us": round(mm["avg_launch_us"], 2)}
            ab = append_bench(dw.kv_cache, NB, bs, H, D, None, None, dev)
            modes[name]["append"] = {k: ab[k] for k in ("per_layer_calls_hip_graph", "one_launch_all_layers")}
            if mono:
                modes["pack_probes_one_allocation"] = pack_chain_probes(sw, tabs, payload, dev)
            release(sw, dw)
            del tabs
        if weights is not None:
            # the reference's layout again, but with nothing allocated before the pools (what a process that only
            # allocates pools gets; not fresh here: this process has allocated and freed other pools before)
            weights = None
            torch.cuda.empty_cache()
            sw, dw = make_workers(NB, L, bs, H, D, dtype, dev, args.spread, monolithic=args.monolithic)
            tabs = [(s.to(dev), d.to(dev)) for s, d in tables]
            mm = measure_migrate(sw, dw, tabs, max(3, args.steps // 4), 2, payload)
            modes["no_weights_resident"] = {
                "value_GBps": round(mm["value"], 1), "frac": round(mm["value"] / HBM_PEAK_GBPS, 4),
                "pack_GBps": round(mm["pack_GBps"], 1), "unpack_GBps": round(mm["unpack_GBps"], 1),
                "note": "in a fresh process (--weights-gib 0) this layout measures 6.07-6.09 TB/s (unpack 5.93-5.97)"}
            release(sw, dw)
            del tabs
        modes["what"] = ("the headline workload on pools allocated differently: 'one_allocation_per_pool' is "
                         "init_kvcache's default (spread_stripes=0), 'four_stripes_per_pool' is init_kvcache("
                         "spread_stripes=4): the layers in 4 pieces pushed apart in device memory with temporary spacer "
                         "allocations. The headline itself runs on " + layout_name(args))
        extra["allocation_modes"] = modes
    weights = None
    torch.cuda.empty_cache()
    if "cfg1" in sections:
        extra["cfg1_latency"] = cfg1_latency(dev)
    if "fp8" in sections:
        w8, g8 = weights_placeholder(args, LLAMA_70B_FP8_WEIGHT_BYTES, dev)
        extra["fp8_70b_shape"] = fp8_shape(dev, args.spread, args.monolithic)
        extra["fp8_70b_shape"]["allocated_before_the_pools_GiB"] = g8
        del w8
        torch.cuda.empty_cache()
    if "rebalance" in sections:
        w5, g5 = weights_placeholder(args, QWEN2_7B_WEIGHT_BYTES, dev)
        extra["rebalance_200GB"] = rebalance(dev)
        extra["rebalance_200GB"]["allocated_before_the_pool_GiB"] = g5
        del w5
        torch.cuda.empty_cache()
    if "swap" in sections:
        extra["swap_pcie"] = swap_bench(dev)

    result = {
        "metric": "KV pack+unpack GB/s",
        "value": round(m["value"], 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(m["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "pct_hbm_peak": round(100.0 * m["value"] / HBM_PEAK_GBPS, 2),
        "config": {
            "workload": "qwen2_7b_migrate: 28 layers x [2,%d,16,4,128] bf16 x 2 pools, %d requests (%d blocks, "
                        "%.2f GB payload), 32 per-request packs, then 32 per-request unpacks under different block tables"
                        % (NB, len(tables), total_blocks, payload / 1e9),
            "num_layers": L, "num_blocks": NB, "block_size": bs, "kv_heads": H, "head_dim": D,
            "requests": len(tables), "blocks_moved": total_blocks, "algorithmic_bytes_per_step": bytes_per_step,
            "pool_allocation": layout_name(args) + " (extra.allocation_modes has the other layouts)",
            "allocated_before_the_pools": ("%.3f GiB standing for the model's weights (Qwen2-7B, bf16): the reference's "
                                           "worker loads the model, then sizes and allocates its pool "
                                           "(elasticmm/engine/v0/worker.py:256, :271-394); --weights-gib 0 allocates the "
                                           "pools first" % weights_gib) if weights_gib else "nothing (--weights-gib 0)",
        },
        "roofline": roofline,
        "extra": extra,
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(tables, L, bs, H, D, dtype)
        result["cpu_baseline"]["append"] = cpu_baseline_append()
        result["cpu_baseline"]["cfg1"] = cpu_baseline_cfg1()
    print(json.dumps(result), flush=True)


# ---------------------------------------------------------------------------------------------- secondary shapes
def batched(src_w, dst_w, dev_tables, payload, L, chunk, NB, dev):
    """One launch for the whole batch, the fused pool-to-pool migrate, copy_blocks, plain-copy yardsticks."""
    from elasticmm_amd import kv_ops

    out = {}
    sp, dp = src_w.pool, dst_w.pool
    all_si = torch.cat([s for s, _ in dev_tables])
    all_di = torch.cat([d for _, d in dev_tables])
    buf = torch.empty(sp.packed_shape(all_si.numel()), dtype=sp.dtype, device=dev)
    med, _ = timed(lambda: kv_ops.kv_pack(sp, all_si, out=buf), 10)
    out["batched_pack"] = rec(2 * payload, med, 1, "emm_block_move_kernel<pack, plain order>")
    med, _ = timed(lambda: kv_ops.kv_unpack(dp, all_di, buf), 10)
    out["batched_unpack"] = rec(2 * payload, med, 1, "emm_block_move_kernel<unpack, grouped order>")
    med, _ = timed(lambda: kv_ops.kv_migrate(sp, all_si, dp, all_di), 10)
    out["fused_migrate"] = rec(2 * payload, med, 1, "emm_block_move_kernel<pool to pool, runs order>",
                               note="replaces a pack and an unpack: half their traffic")

    def interleaved():
        for si, di in dev_tables:
            dst_w.write_kv_blocks(di, src_w.extract_kv_blocks(si))

    med, _ = timed(interleaved, 5)
    out["per_request_pack_then_unpack_interleaved"] = rec(
        4 * payload, med, 2 * len(dev_tables), note="each buffer unpacked right after its pack: partly read back from "
                                                    "the 256 MB last-level cache, not the headline")
    # per-request launches alternating over two streams of the same priority: the drain of one launch overlaps the
    # ramp of the next (the kernels take the current stream, so a caller can do this with the product as it is)
    bufs2 = [torch.empty(sp.packed_shape(s.numel()), dtype=sp.dtype, device=dev) for s, _ in dev_tables]
    side = torch.cuda.Stream()

    def fan_out(fn):
        main = torch.cuda.current_stream()
        side.wait_stream(main)
        for i, (tab, b) in enumerate(zip(dev_tables, bufs2)):
            if i & 1:
                with torch.cuda.stream(side):
                    fn(tab, b)
            else:
                fn(tab, b)
        main.wait_stream(side)

    med_p, _ = timed(lambda: fan_out(lambda tab, b: kv_ops.kv_pack(sp, tab[0], out=b)), 10)
    med_u, _ = timed(lambda: fan_out(lambda tab, b: kv_ops.kv_unpack(dp, tab[1], b)), 10)
    med_p1, _ = timed(lambda: [kv_ops.kv_pack(sp, tab[0], out=b) for tab, b in zip(dev_tables, bufs2)], 10)
    med_u1, _ = timed(lambda: [kv_ops.kv_unpack(dp, tab[1], b) for tab, b in zip(dev_tables, bufs2)], 10)
    out["per_request_two_streams"] = {
        "pack": rec(2 * payload, med_p, len(dev_tables)), "unpack": rec(2 * payload, med_u, len(dev_tables)),
        "pack_one_stream": rec(2 * payload, med_p1, len(dev_tables)),
        "unpack_one_stream": rec(2 * payload, med_u1, len(dev_tables)),
        "note": "the same 32 per-request launches alternating over two streams against one stream, same buffers"}
    del bufs2
    flat = buf.view(-1)
    other = torch.empty_like(flat)
    med, _ = timed(lambda: kv_ops.stream_copy(flat, other), 10)
    out["plain_copy_same_engine"] = rec(2 * payload, med, 1, "emm_stream_copy_kernel")
    med, _ = timed(lambda: other.copy_(flat), 10)
    out["torch_copy"] = rec(2 * payload, med, 1, "torch.Tensor.copy_")
    del other, buf
    # copy_blocks: half of the batch's blocks to free blocks of the same pool
    P = all_si.numel() // 2
    used = torch.zeros(NB, dtype=torch.bool, device=dev)
    used[all_si] = True
    free = (~used).nonzero().squeeze(1)
    if free.numel() >= P:
        mapping = torch.stack([all_si[:P], free[:P]], 1).contiguous()
        med, _ = timed(lambda: kv_ops.copy_blocks(sp, mapping), 10)
        out["copy_blocks"] = rec(2 * P * L * 2 * chunk, med, 1, "emm_block_move_kernel<pool to pool, pairs>")
    return out


def ceilings(src_w, dst_w, dev_tables, payload, dev):
    """Measured ceilings of this memory system for the access patterns of pack and unpack, each half on its own
    (kernels of the hooks build with the grid of pack / unpack: one 4 KiB tile per 256-thread workgroup):
    sequential read, sequential write, gathered read of the batch's 16 KiB chunks from the source pool,
    scattered write of them into the destination pool. Rates are bytes touched / time (one direction)."""
    from elasticmm_amd import _lib

    hooks = _lib.load_hooks()
    sp, dp = src_w.pool, dst_w.pool
    all_si = torch.cat([s for s, _ in dev_tables]).contiguous()
    all_di = torch.cat([d for _, d in dev_tables]).contiguous()
    n = all_si.numel()
    lin = torch.empty(payload, dtype=torch.uint8, device=dev).random_(0, 255)
    sink = torch.zeros(1024, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    stab, dtab = _lib.ptr_table(sp.ptrs), _lib.ptr_table(dp.ptrs)

    def probe(kind, table, idx):
        rc = hooks.emm_hook_probe(kind, table, sp.num_layers, sp.num_kv, sp.num_blocks, sp.chunk_bytes,
                                  idx.data_ptr() if idx is not None else None, n, lin.data_ptr(), sink.data_ptr(), stream)
        if rc != 0:
            raise RuntimeError(hooks.emm_last_error().decode())

    out = {}
    for name, kind, table, idx in (("sequential_read", _lib.EMM_PROBE_SEQ_READ, None, None),
                                   ("sequential_write", _lib.EMM_PROBE_SEQ_WRITE, None, None),
                                   ("gather_read_16KiB_chunks", _lib.EMM_PROBE_GATHER_READ, stab, all_si),
                                   ("scatter_write_16KiB_chunks", _lib.EMM_PROBE_SCATTER_WRITE, dtab, all_di)):
        med, _ = timed(lambda: probe(kind, table, idx), 10)
        out[name] = rec(payload, med, 1, "emm_probe_kernel")
    # what fetching the block id costs a pack: the same gather with ids computed in registers, and the whole pack
    # (gathered read + sequential write, 2 x payload) with fetched and with computed ids
    med, _ = timed(lambda: probe(_lib.EMM_PROBE_GATHER_READ_COMPUTED_IDS, stab, all_si), 10)
    out["gather_read_computed_ids"] = rec(payload, med, 1, "emm_probe_kernel")
    med, _ = timed(lambda: probe(_lib.EMM_PROBE_PACK, stab, all_si), 10)
    out["pack_probe_fetched_ids"] = rec(2 * payload, med, 1, "emm_probe_kernel")
    med, _ = timed(lambda: probe(_lib.EMM_PROBE_PACK_COMPUTED_IDS, stab, all_si), 10)
    out["pack_probe_computed_ids"] = rec(2 * payload, med, 1, "emm_probe_kernel")
    r, w = out["sequential_read"]["GBps"], out["sequential_write"]["GBps"]
    g, s = out["gather_read_16KiB_chunks"]["GBps"], out["scatter_write_16KiB_chunks"]["GBps"]
    out["harmonic_seq_read_seq_write"] = round(2 / (1 / r + 1 / w), 1)
    out["harmonic_gather_read_seq_write"] = round(2 / (1 / g + 1 / w), 1)
    out["harmonic_seq_read_scatter_write"] = round(2 / (1 / r + 1 / s), 1)
    out["note"] = ("a copy alternates reads and writes on the same channels and stays below the harmonic mean of its two "
                   "halves (compare plain_copy_same_engine with harmonic_seq_read_seq_write); the scatter probe overwrote "
                   "the destination blocks of the batch")
    del lin
    return out


def pack_chain_probes(src_w, dev_tables, payload, dev):
    """What the scalar fetches in front of a pack's data loads cost (whole batch in one launch, probe kernels of the hooks
    build on a pool in one allocation): ids and plane bases fetched (the product kernel's chain), ids computed in registers,
    and ids and plane bases both computed — no load at all before the data."""
    from elasticmm_amd import _lib

    hooks = _lib.load_hooks()
    sp = src_w.pool
    all_si = torch.cat([s for s, _ in dev_tables]).contiguous()
    n = all_si.numel()
    lin = torch.empty(payload, dtype=torch.uint8, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    stab = _lib.ptr_table(sp.ptrs)

    def probe(kind):
        rc = hooks.emm_hook_probe(kind, stab, sp.num_layers, sp.num_kv, sp.num_blocks, sp.chunk_bytes, all_si.data_ptr(), n,
                                  lin.data_ptr(), None, stream)
        if rc != 0:
            raise RuntimeError(hooks.emm_last_error().decode())

    out = {}
    for name, kind in (("ids_and_plane_bases_fetched", _lib.EMM_PROBE_PACK), ("ids_computed", _lib.EMM_PROBE_PACK_COMPUTED_IDS),
                       ("nothing_fetched", _lib.EMM_PROBE_PACK_NOTHING_FETCHED)):
        med, _ = timed(lambda: probe(kind), 10)
        out[name] = rec(2 * payload, med, 1, "emm_probe_kernel")
    del lin
    return out


def placement(src_w, dst_w, dev_tables, payload, dev):
    """Where an allocation lands in device memory decides how fast scattered writes into it are, and that follows what
    the device's memory manager handed out and took back before (same virtual addresses every time): the batch's per-request unpacks into the
    destination pool and, from the same buffers, into the source pool of this process; and a scatter-write / gather-read
    probe (hooks build) of the batch's chunks into every layer — every allocation — of both pools by itself."""
    from elasticmm_amd import _lib, kv_ops

    hooks = _lib.load_hooks()
    sp, dp = src_w.pool, dst_w.pool
    bufs = [kv_ops.kv_pack(sp, s) for s, _ in dev_tables]
    out = {}
    for name, pool in (("unpack_into_destination_pool", dp), ("unpack_into_source_pool", sp)):
        med, _ = timed(lambda: [kv_ops.kv_unpack(pool, d, b) for (_, d), b in zip(dev_tables, bufs)], 10)
        out[name] = rec(2 * payload, med, len(bufs), "emm_block_move_kernel<unpack>")
    del bufs
    all_di = torch.cat([d for _, d in dev_tables]).contiguous()
    n = all_di.numel()
    lin = torch.empty(sp.num_kv * n * sp.chunk_bytes, dtype=torch.uint8, device=dev)
    sink = torch.zeros(1024, dtype=torch.int32, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    layer_bytes = sp.num_kv * n * sp.chunk_bytes
    for pname, pool in (("destination_pool", dp), ("source_pool", sp)):
        for kname, kind in (("scatter_write", _lib.EMM_PROBE_SCATTER_WRITE), ("gather_read", _lib.EMM_PROBE_GATHER_READ)):
            rates = []
            for l in range(pool.num_layers):
                tab = _lib.ptr_table(pool.ptrs[l:l + 1])

                def probe():
                    rc = hooks.emm_hook_probe(kind, tab, 1, pool.num_kv, pool.num_blocks, pool.chunk_bytes, all_di.data_ptr(),
                                              n, lin.data_ptr(), sink.data_ptr(), stream)
                    if rc != 0:
                        raise RuntimeError(hooks.emm_last_error().decode())

                med, _ = timed(probe, 5, warmup=1)
                rates.append(round(layer_bytes / med / 1e6))
            out["%s_%s_GBps_per_layer" % (pname, kname)] = rates
    out["note"] = ("each layer is an allocation of its own; the probes touch the batch's %d chunks of 16 KiB in both planes of "
                   "one layer per launch (%.0f MB)" % (n, layer_bytes / 1e6))
    return out


def reallocation_cycles(args, tables, NB, L, bs, H, D, dtype, payload, dev, cycles=4):
    """The headline workload on pools that this process frees and allocates again, cycle after cycle (same layout, same
    virtual addresses; the memory goes back to the driver in between). What the driver hands out changes with every
    cycle of allocating and freeing — in this process and in the processes that ran on the device before — and with it
    the rate of scattered writes into the pools: a fresh device gives its first process the slowest placement seen,
    after three cycles of this size the figures settle."""
    out = []
    for _ in range(cycles):
        sw, dw = make_workers(NB, L, bs, H, D, dtype, dev, args.spread, monolithic=args.monolithic)
        tabs = [(s.to(dev), d.to(dev)) for s, d in tables]
        mm = measure_migrate(sw, dw, tabs, 5, 2, payload)
        bufs = [sw.extract_kv_blocks(s) for s, _ in tabs]
        med, _ = timed(lambda: [sw.write_kv_blocks(d, b) for (_, d), b in zip(tabs, bufs)], 5)
        out.append({"value_GBps": round(mm["value"], 1), "pack_GBps": round(mm["pack_GBps"], 1),
                    "unpack_GBps": round(mm["unpack_GBps"], 1),
                    "unpack_into_source_pool_GBps": round(2 * payload / med / 1e6, 1)})
        del bufs, tabs
        release(sw, dw)
        del sw, dw
        torch.cuda.empty_cache()
    return out


def pack_variants(src_w, dev_tables, payload, dev):
    """The pack through the other kernel shapes kept in the hooks build (csrc/emm_kv_hooks.h: two / four tiles per
    workgroup, loads straight into LDS, loader and storer waves), next to the product kernel: the whole batch in one
    launch, and the 32 per-request launches."""
    from elasticmm_amd import _lib, kv_ops

    hooks = _lib.load_hooks()
    sp = src_w.pool
    all_si = torch.cat([s for s, _ in dev_tables]).contiguous()
    n = all_si.numel()
    buf = torch.empty(sp.packed_shape(n), dtype=sp.dtype, device=dev)
    stab = _lib.ptr_table(sp.ptrs)
    stream = torch.cuda.current_stream().cuda_stream

    def variant(code, idx, out):
        rc = hooks.emm_hook_pack_variant(code, stab, sp.num_layers, sp.num_kv, sp.num_blocks, sp.chunk_bytes,
                                         idx.data_ptr(), idx.numel(), out.data_ptr(), stream)
        if rc != 0:
            raise RuntimeError(hooks.emm_last_error().decode())

    bufs = [torch.empty(sp.packed_shape(s.numel()), dtype=sp.dtype, device=dev) for s, _ in dev_tables]
    out = {}
    med, _ = timed(lambda: kv_ops.kv_pack(sp, all_si, out=buf), 10)
    med_r, _ = timed(lambda: [kv_ops.kv_pack(sp, s, out=b) for (s, _), b in zip(dev_tables, bufs)], 10)
    out["product_kernel"] = {"whole_batch": rec(2 * payload, med, 1, "emm_block_move_kernel<pack>"),
                             "per_request": rec(2 * payload, med_r, len(bufs), "emm_block_move_kernel<pack>")}
    want = buf.clone()
    for name, code in _lib.EMM_PACK_VARIANTS.items():
        buf.zero_()
        med, _ = timed(lambda: variant(code, all_si, buf), 10)
        same = bool(torch.equal(buf, want))
        med_r, _ = timed(lambda: [variant(code, s, b) for (s, _), b in zip(dev_tables, bufs)], 10)
        out[name] = {"whole_batch": rec(2 * payload, med, 1, "emm_pack_variant_kernel<%d>" % code),
                     "per_request": rec(2 * payload, med_r, len(bufs), "emm_pack_variant_kernel<%d>" % code),
                     "same_result_as_product": same}
    return out


def paged_append_bench(kv, NB, bs, H, D, dev, T=8448, decode=256, k_scales=None, v_scales=None):
    """The same step appended into the paged-attention layout (key [NB,H,D/x,bs,x], value [NB,H,D,bs],
    x = 16 bytes of cache elements, viewed over the same pool memory): `decode` single tokens in random
    blocks, then one prompt of T - decode tokens that fills blocks in order (its blocks start off the
    16-token grid of the token list). Bytes per token and layer: the K and V rows read (16-bit) and written
    (the cache's element size), as for the flash layout. With scales the cache is fp8 (quantising append)."""
    from elasticmm_amd import cache_ops

    L = len(kv)
    ce = kv[0].element_size()
    fp8 = k_scales is not None
    cache_dtype = "fp8" if fp8 else "auto"
    kernel = "emm_append_paged_kernel" if fp8 else "emm_append_paged_wave_kernel"
    x = 16 // ce
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
    step_bytes = L * (T * 2 * H * D * (2 + ce) + 8 * T)
    ks = [k_scales[l:l + 1] for l in range(L)] if fp8 else [None] * L
    vs = [v_scales[l:l + 1] for l in range(L)] if fp8 else [None] * L

    def per_layer():
        for l in range(L):
            cache_ops.reshape_and_cache(keys[l], values[l], kcs[l], vcs[l], slots, cache_dtype, ks[l], vs[l])

    def entry(ms, launches):
        return rec(step_bytes, ms, launches, kernel, tokens_per_s=round(T / (ms * 1e-3)))

    res = {"T": T, "decode_tokens": decode, "layers": L}
    med, _ = timed(per_layer, 20)
    res["per_layer_calls_eager"] = entry(med, L)
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        per_layer()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(graph):
        per_layer()
    med, _ = timed(graph.replay, 20)
    res["per_layer_calls_hip_graph"] = entry(med, L)
    plan = cache_ops.paged_layered_append(keys, values, kcs, vcs, cache_dtype, k_scales, v_scales)
    med, _ = timed(lambda: plan(slots), 20)
    res["one_launch_all_layers"] = entry(med, 1)
    # a decode-only step: every token alone in its block (each 2-byte V element and each 16-byte K piece
    # lands in a cache line of its own, so the memory system rewrites the token's whole block region)
    Td = 256
    dplan = cache_ops.paged_layered_append([k[:Td] for k in keys], [v[:Td] for v in values], kcs, vcs,
                                           cache_dtype, k_scales, v_scales)
    dslots = dec[:Td].contiguous() if decode >= Td else slots[:Td].contiguous()
    med, _ = timed(lambda: dplan(dslots), 20)
    res["decode_only_256_tokens_one_launch"] = rec(L * Td * 2 * H * D * (2 + ce), med, 1, kernel,
                                                   tokens_per_s=round(Td / (med * 1e-3)))

    def decode_per_layer():
        for l in range(L):
            cache_ops.reshape_and_cache(keys[l][:Td], values[l][:Td], kcs[l], vcs[l], dslots, cache_dtype, ks[l], vs[l])

    def decode_graph():
        dgraph = torch.cuda.CUDAGraph()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            decode_per_layer()
        torch.cuda.current_stream().wait_stream(side)
        with torch.cuda.graph(dgraph):
            decode_per_layer()
        med, _ = timed(dgraph.replay, 20)
        res["decode_step_256_tokens_per_layer_hip_graph"] = rec(L * Td * 2 * H * D * (2 + ce), med, L, kernel,
                                                                tokens_per_s=round(Td / (med * 1e-3)))

    if fp8:
        decode_graph()
        return res

    # the flash layout behind a head-major pool [NB, H, bs, D], handed over as the permuted view vLLM builds: the
    # strided append kernel, all layers in one launch
    from elasticmm_amd import kv_ops
    hk = [kv[l][0].view(NB, H, bs, D).permute(0, 2, 1, 3) for l in range(L)]
    hv = [kv[l][1].view(NB, H, bs, D).permute(0, 2, 1, 3) for l in range(L)]
    def head_major():
        kv_ops.reshape_and_cache_strided(keys, values, hk, hv, slots)

    hgraph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        head_major()
    torch.cuda.current_stream().wait_stream(side)
    with torch.cuda.graph(hgraph):
        head_major()
    med, _ = timed(hgraph.replay, 20)  # replayed: the Python call checks 4 x 28 tensors before its one launch
    res["head_major_pool_one_launch_all_layers"] = rec(step_bytes, med, 1, "emm_append_strided_kernel",
                                                       tokens_per_s=round(T / (med * 1e-3)))
    med, _ = timed(head_major, 20)
    res["head_major_pool_one_launch_all_layers"]["eager_call_us"] = round(med * 1e3, 1)

    decode_graph()
    return res


APPEND_CONTEXT = True  # main() clears it for --no-append-context


def append_bench(kv, NB, bs, H, D, k_scales, v_scales, dev, T=8448):
    """reshape_and_cache for one step: 256 decode tokens + one 8192-token prefill chunk, slots random
    over the pool, 5 % padded (-1). Three ways of issuing it: the vLLM-shaped call once per layer
    (eager Python), the same L launches replayed from a HIP graph, and one launch for all layers from
    a prepared plan (possible only where every layer's K/V already exists: re-ingest, prefix load — not
    a model forward, which produces layer l+1's K/V after layer l's append). tokens/s = valid tokens /
    time of all layers. `launch_bound_yardsticks` replays, from the same kind of graph, L plain copies
    of one layer's bytes with the library's copy kernel: what a chain of L dependent launches of
    that size costs on this machine with no indirection at all."""
    from elasticmm_amd import cache_ops, kv_ops

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
    kernel = "emm_append_fp8_kernel" if fp8 else "emm_append_kernel"

    def per_layer():
        for l in range(L):
            cache_ops.reshape_and_cache_flash(keys[l], values[l], kv[l][0], kv[l][1], slots, mode, ks[l], vs[l])

    def entry(ms, launches):
        return rec(step_bytes, ms, launches, kernel, tokens_per_s=round(valid / (ms * 1e-3)))

    def graphed(fn):
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()
        torch.cuda.current_stream().wait_stream(side)
        with torch.cuda.graph(graph):
            fn()
        return graph

    res = {"T": T, "valid": valid, "layers": L}
    med, _ = timed(per_layer, 20)
    res["per_layer_calls_eager"] = entry(med, L)
    med, _ = timed(graphed(per_layer).replay, 20)
    res["per_layer_calls_hip_graph"] = entry(med, L)
    plan = cache_ops.layered_append(keys, values, kv, mode, k_scales, v_scales)
    med, _ = timed(lambda: plan(slots), 20)
    res["one_launch_all_layers"] = entry(med, 1)
    # The per-layer launch where it really runs. (1) The same L launches as INDEPENDENT graph nodes: forked over k
    # streams of the same priority inside the capture and joined at the end, so that nothing orders one layer's append
    # after another's (what a runtime could do if the appends of several layers were ready at once). (2) Inside a
    # forward: a kernel of the duration of a layer's other work between two appends (here the QKV projection that
    # produces the K / V the append stores: [T, 3584] x [3584, 4608] bf16), L times, replayed from a graph with and
    # without the appends; the difference per layer is what the forward pays for an append.
    if APPEND_CONTEXT:
        res["in_context"] = append_in_context(keys, values, kv, slots, mode, ks, vs, entry, graphed, step_bytes, valid,
                                              kernel, T, H, D, L, dev, g)
    # a decode step: 256 tokens, one per sequence, per-layer launches from a HIP graph (the most frequent step of a
    # serving loop; 1 MB per launch, so the figure of merit is microseconds per launch against the empty launch)
    Td = 256
    dslots = slots[slots >= 0][:Td].contiguous()
    return _append_bench_tail(res, keys, values, kv, slots, dslots, Td, mode, ks, vs, graphed, kernel, row, step_bytes, L, dev)


def append_in_context(keys, values, kv, slots, mode, ks, vs, entry, graphed, step_bytes, valid, kernel, T, H, D, L, dev, g):
    from elasticmm_amd import cache_ops

    side_streams = [torch.cuda.Stream() for _ in range(3)]

    def forked(k):
        main = torch.cuda.current_stream()
        for st in side_streams[:k - 1]:
            st.wait_stream(main)
        for l in range(L):
            st = main if l % k == 0 else side_streams[l % k - 1]
            with torch.cuda.stream(st):
                cache_ops.reshape_and_cache_flash(keys[l], values[l], kv[l][0], kv[l][1], slots, mode, ks[l], vs[l])
        for st in side_streams[:k - 1]:
            main.wait_stream(st)

    ctx = {}
    for k in (2, 4):
        med, _ = timed(graphed(lambda: forked(k)).replay, 20)
        ctx["independent_graph_nodes_over_%d_streams" % k] = entry(med, L)
    hidden, qkv = 3584, 3584 + 2 * H * D
    xin = torch.randn((T, hidden), device=dev, generator=g).to(torch.bfloat16)
    wqkv = (torch.randn((hidden, qkv), device=dev, generator=g) * 0.02).to(torch.bfloat16)
    yout = torch.empty((T, qkv), dtype=torch.bfloat16, device=dev)

    def forward_like(with_append):
        for l in range(L):
            torch.mm(xin, wqkv, out=yout)
            if with_append:
                cache_ops.reshape_and_cache_flash(keys[l], values[l], kv[l][0], kv[l][1], slots, mode, ks[l], vs[l])

    # the difference of two chains of ~240 us per layer: the two graphs are replayed alternately, round after round, so
    # that clock and temperature drift hits both alike; the figure is the median of the rounds' differences
    g_with, g_without = graphed(lambda: forward_like(True)), graphed(lambda: forward_like(False))
    rounds = []
    for _ in range(9):
        a, _ = timed(g_with.replay, 5, warmup=1)
        b, _ = timed(g_without.replay, 5, warmup=1)
        rounds.append((a, b))
    diffs = sorted((a - b) * 1e3 / L for a, b in rounds)
    marginal_us = diffs[len(diffs) // 2]
    med_with = sorted(a for a, _ in rounds)[len(rounds) // 2]
    med_without = sorted(b for _, b in rounds)[len(rounds) // 2]
    ctx["between_projection_kernels"] = {
        "filler": "torch.mm [%d, %d] x [%d, %d] bf16 per layer" % (T, hidden, hidden, qkv),
        "filler_us_per_layer": round(med_without * 1e3 / L, 2),
        "with_append_us_per_layer": round(med_with * 1e3 / L, 2),
        "append_marginal_us_per_layer": round(marginal_us, 2),
        "append_marginal_us_per_layer_rounds_min_max": [round(diffs[0], 2), round(diffs[-1], 2)],
        "append_marginal": rec(step_bytes, marginal_us * L * 1e-3, L, kernel, tokens_per_s=round(valid / (marginal_us * L * 1e-6))),
    }
    del xin, wqkv, yout
    return ctx


def _append_bench_tail(res, keys, values, kv, slots, dslots, Td, mode, ks, vs, graphed, kernel, row, step_bytes, L, dev):
    from elasticmm_amd import cache_ops, kv_ops

    def decode_per_layer():
        for l in range(L):
            cache_ops.reshape_and_cache_flash(keys[l][:Td], values[l][:Td], kv[l][0], kv[l][1], dslots, mode, ks[l], vs[l])

    med, _ = timed(graphed(decode_per_layer).replay, 20)
    res["decode_step_256_tokens_per_layer_hip_graph"] = rec(
        L * (Td * 2 * row * (2 + kv[0].element_size()) + 8 * Td), med, L, kernel, tokens_per_s=round(Td / (med * 1e-3)))
    # yardstick: L dependent launches of a plain copy of the same bytes per layer
    layer_bytes = step_bytes // L
    half = layer_bytes // 2 // 4096 * 4096
    srcs = [torch.empty(half, dtype=torch.uint8, device=dev).random_(0, 255) for _ in range(L)]
    dsts = [torch.empty(half, dtype=torch.uint8, device=dev) for _ in range(L)]

    def copies():
        for l in range(L):
            kv_ops.stream_copy(srcs[l], dsts[l])

    med, _ = timed(graphed(copies).replay, 20)
    from elasticmm_amd import _lib
    hooks = _lib.load_hooks()

    def empties():
        stream = torch.cuda.current_stream().cuda_stream
        for _ in range(L):
            hooks.emm_hook_empty_launch(stream)

    med_e, _ = timed(graphed(empties).replay, 20)
    res["launch_bound_yardsticks"] = {
        "plain_copy_of_one_layers_bytes_per_launch_hip_graph": rec(2 * half * L, med, L, "emm_stream_copy_kernel"),
        "empty_kernel_per_launch_hip_graph_us": round(med_e * 1e3 / L, 2),
        "note": "chains of L dependent launches replayed from a HIP graph: a plain copy of one layer's bytes per launch "
                "(no slot indirection) and a kernel that does nothing; the per-layer append cannot be faster than the "
                "first, and no chain of launches than the second plus the bytes at copy speed"}
    return res


def latency_case(dev, L, NB, bs, H, D, dtype, n):
    """Latency of one extract_kv_blocks + one write_kv_blocks for a request of `n` blocks: back to back in a chain
    (the GPU never idles), and one isolated call with the device idle before and after (host launch + kernels +
    completion). Disjoint block tables are cycled so that consecutive calls touch different blocks."""
    from elasticmm_amd.worker import KVWorker

    sw, dw = KVWorker(0, "cuda:0", bs), KVWorker(1, "cuda:0", bs)
    for w in (sw, dw):
        w.init_kvcache(NB, num_layers=L, num_kv_heads=H, head_size=D, dtype=dtype, monolithic=False)
    for t in sw.kv_cache:
        t.normal_()
    g = torch.Generator().manual_seed(0)
    sp, dp = torch.randperm(NB, generator=g), torch.randperm(NB, generator=torch.Generator().manual_seed(1))
    cycle = min(32, NB // n)
    tabs = [(sp[i * n:(i + 1) * n].to(dev), dp[i * n:(i + 1) * n].to(dev)) for i in range(cycle)]
    lists = [(s.tolist(), d.tolist()) for s, d in tabs]
    nbytes = 4 * n * L * 2 * bs * H * D * torch.empty((), dtype=dtype).element_size()
    state = {"i": 0}

    def one(tables):
        s, d = tables[state["i"] % cycle]
        state["i"] += 1
        dw.write_kv_blocks(d, sw.extract_kv_blocks(s))

    def many(tables, k=32):
        for _ in range(k):
            one(tables)

    def isolated(tables):
        torch.cuda.synchronize()
        ts = []
        for _ in range(50):
            t0 = time.perf_counter()
            one(tables)
            torch.cuda.synchronize()
            ts.append(time.perf_counter() - t0)
        ts.sort()
        return round(ts[len(ts) // 2] * 1e6, 1)

    med, _ = timed(lambda: many(tabs), 10)
    out = {"device_tables": rec(nbytes * 32, med, 64, "emm_block_move_kernel", us_per_pack_plus_unpack=round(med * 1e3 / 32, 2))}
    med, _ = timed(lambda: many(lists), 10)
    out["list_indices"] = rec(nbytes * 32, med, 64, "emm_block_move_kernel", us_per_pack_plus_unpack=round(med * 1e3 / 32, 2))
    out["isolated_call_wall_us"] = isolated(tabs)
    out["isolated_call_wall_us_list_indices"] = isolated(lists)
    out["bytes_per_pack_plus_unpack"] = nbytes
    release(sw, dw)
    return out


def cfg1_latency(dev):
    """Small requests: config 1 (4 layers x [2,1024,16,8,128] fp16, one request of 32 blocks, 8 MiB buffer) and the
    reference's own typical transfer (15 blocks = 234 tokens, elasticmm/engine/v0/README.md:38-47) on the Qwen2-7B
    layout (28 layers x [2,NB,16,4,128] bf16: 13.1 MiB per request). The floor under an isolated call is what two
    kernels that do nothing cost the same way (launch, launch, synchronise)."""
    from elasticmm_amd import _lib

    out = latency_case(dev, 4, 1024, 16, 8, 128, torch.float16, 32)
    out["typical_request_15_blocks_qwen2_7b_layout"] = latency_case(dev, 28, 2048, 16, 4, 128, torch.bfloat16, 15)
    hooks = _lib.load_hooks()
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    ts = []
    for _ in range(50):
        t0 = time.perf_counter()
        hooks.emm_hook_empty_launch(stream)
        hooks.emm_hook_empty_launch(stream)
        torch.cuda.synchronize()
        ts.append(time.perf_counter() - t0)
    ts.sort()
    out["two_empty_kernels_isolated_wall_us"] = round(ts[len(ts) // 2] * 1e6, 1)
    return out


def fp8_shape(dev, spread=0, monolithic=False):
    """Config 4: 80 layers x [2, NB, 16, 8, 128] e4m3, 64 requests of U{1024..8192} tokens: pack / unpack of fp8
    bytes, the quantising append (bf16 -> fp8), the dequantising unpack (fp8 -> bf16 pool)."""
    from elasticmm_amd import kv_ops
    from elasticmm_amd.kv_ops import PoolView
    from elasticmm_amd.worker import allocate_layers_spread

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

    def make_pool(dtype):
        shape = (2, NB, bs, H, D)
        if spread > 1:
            return allocate_layers_spread(L, shape, dtype, dev, spread)
        if monolithic:
            return list(torch.empty((L,) + shape, dtype=dtype, device=dev).unbind(0))
        return [torch.empty(shape, dtype=dtype, device=dev) for _ in range(L)]  # the reference's layout

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
    out = {"layers": L, "pool_blocks": NB, "requests": 64, "blocks": total, "payload_GB": round(payload / 1e9, 2),
           "pool_allocation": "spread_stripes=%d" % spread if spread > 1 else "one allocation per pool" if monolithic
           else "one torch.empty per layer",
           "pack": rec(2 * payload, ts_pack, 64, "emm_block_move_kernel<pack>"),
           "unpack": rec(2 * payload, ts_unpack, 64, "emm_block_move_kernel<unpack>"),
           "pack_plus_unpack": rec(4 * payload, ts_pack + ts_unpack, 128, "emm_block_move_kernel")}
    out["append"] = append_bench(src, NB, bs, H, D, k_scales, v_scales, dev)
    out["append_paged_layout"] = paged_append_bench(src, NB, bs, H, D, dev, k_scales=k_scales, v_scales=v_scales)
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
    out["dequant_unpack"] = rec(3 * pay, t_dq, 16, "emm_unpack_dequant_fp8_kernel",
                                note="1 fp8 byte read + 2 bf16 bytes written per element")
    del src, sp, dq, dqp
    torch.cuda.empty_cache()
    return out


def swap_bench(dev):
    """GPU <-> CPU swap (pinned host pool, kernels read / write it over PCIe): Qwen2-7B layout."""
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
    out = {"blocks": nsw, "GB": round(sw_bytes / 1e9, 3), "bound": "PCIe, not HBM",
           "swap_out_GBps": round(sw_bytes / t_out / 1e9, 1), "swap_in_GBps": round(sw_bytes / t_in / 1e9, 1),
           "contiguous_memcpy_d2h_GBps": round(sw_bytes / t_d2h / 1e9, 1),
           "contiguous_memcpy_h2d_GBps": round(sw_bytes / t_h2d / 1e9, 1)}
    del w, stage_g, stage_c
    torch.cuda.empty_cache()
    return out


def rebalance(dev):
    """Config 5: ~200 GB bf16 pool in the Qwen2-7B layout, copy_blocks moves 50 % of the live half to disjoint free
    blocks; the vision-embedding gather (128 images, 64..2304 patches x 3584 bf16) alone, interleaved with
    copy_blocks on the same stream, and on a second stream next to it."""
    from elasticmm_amd import kv_ops
    from elasticmm_amd.kv_ops import PoolView

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
    copy_bytes = 2 * P * L * 2 * chunk
    med, _ = timed(lambda: kv_ops.copy_blocks(pv, mapping), 5, warmup=1)
    ok = bool(torch.equal(pool[3][:, mapping[:1000, 1]], pool[3][:, mapping[:1000, 0]]))
    out = {"pool_GB": round(pool.numel() * 2 / 1e9, 1), "pairs": P, "spot_check": ok,
           "copy_blocks": rec(copy_bytes, med, 1, "emm_block_move_kernel<pool to pool, pairs>")}
    imgs = torch.randint(64, 2305, (128,), generator=g).tolist()
    embeds = [torch.randn((p_, 3584), device=dev).to(torch.bfloat16) for p_ in imgs]
    vis_bytes = 2 * sum(imgs) * 3584 * 2
    outbuf = torch.empty((sum(imgs), 3584), dtype=torch.bfloat16, device=dev)
    vc = {"images": 128, "rows": sum(imgs)}
    # Four calls per timed region: the host prepares the next call (pointer table of 128 segments) while the
    # previous launch runs, as in a serving loop; one isolated call leaves the GPU idle for that time and is
    # reported next to it.
    def chain4(fn):
        med4, _ = timed(lambda: (fn(), fn(), fn(), fn()), 10)
        return med4 / 4
    med1, _ = timed(lambda: kv_ops.concat_rows(embeds, out=outbuf), 10)
    vc["tensor_list"] = rec(vis_bytes, chain4(lambda: kv_ops.concat_rows(embeds, out=outbuf)), 1, "emm_concat_rows_kernel")
    vc["tensor_list"]["isolated_call_ms"] = round(med1, 4)
    # the same gather from segments prepared when the embeddings entered the cache (what
    # KVWorker.gather_vision_embeddings does): the host reads two fields per image instead of the tensors
    prepared = [kv_ops.RowSource(e) for e in embeds]
    med1, _ = timed(lambda: kv_ops.concat_row_sources(prepared, out=outbuf), 10)
    vc["prepared_segments"] = rec(vis_bytes, chain4(lambda: kv_ops.concat_row_sources(prepared, out=outbuf)), 1,
                                  "emm_concat_rows_kernel")
    vc["prepared_segments"]["isolated_call_ms"] = round(med1, 4)
    vc["torch_cat"] = rec(vis_bytes, chain4(lambda: torch.cat(embeds, 0, out=outbuf)), 1, "torch.cat")
    out["vision_concat"] = vc
    parts = 8
    row_off = [0]
    for k in range(parts):
        row_off.append(row_off[-1] + sum(imgs[k * 16:(k + 1) * 16]))
    tot = 2 * (P // parts) * parts * L * 2 * chunk + vis_bytes

    def interleaved():
        for k in range(parts):
            kv_ops.copy_blocks(pv, mapping[k * (P // parts):(k + 1) * (P // parts)])
            kv_ops.concat_row_sources(prepared[k * 16:(k + 1) * 16], out=outbuf[row_off[k]:row_off[k + 1]])

    med, _ = timed(interleaved, 3, warmup=1)
    out["interleaved_same_stream"] = rec(tot, med, 2 * parts, note="8 x (copy_blocks of an eighth of the pairs, then "
                                                                   "the gather of 16 images), alternating on one stream")
    side = torch.cuda.Stream()  # default priority

    def two_streams():
        cur = torch.cuda.current_stream()
        side.wait_stream(cur)
        with torch.cuda.stream(side):
            for k in range(parts):
                kv_ops.concat_row_sources(prepared[k * 16:(k + 1) * 16], out=outbuf[row_off[k]:row_off[k + 1]])
        for k in range(parts):
            kv_ops.copy_blocks(pv, mapping[k * (P // parts):(k + 1) * (P // parts)])
        cur.wait_stream(side)

    med, _ = timed(two_streams, 3, warmup=1)
    out["interleaved_two_streams"] = rec(tot, med, 2 * parts, note="the same launches with the gathers on a second "
                                                                   "stream of the same priority, joined at the end")
    del pool, pv, embeds, prepared, outbuf
    torch.cuda.empty_cache()
    return out


if __name__ == "__main__":
    main()
