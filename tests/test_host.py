"""Host-side logic of the drop-in surface (no GPU needed)."""
import numpy as np
import pytest
import torch

from elasticmm_amd import kv_ops
from elasticmm_amd.block_manager import BlockLocation, BlockManager, VisionBlockManager
from elasticmm_amd.kv_transfer import KVTransferManager, TransferMethod
from elasticmm_amd.worker import KVWorker, LoopbackLink


def test_block_index_tensor_follows_torch_indexing_rules():
    cpu = torch.device("cpu")
    t = kv_ops.block_index_tensor([3, 0, -1, -8], 8, cpu)
    assert t.dtype == torch.long and t.tolist() == [3, 0, 7, 0]
    x = torch.arange(8)
    assert torch.equal(x[torch.tensor([3, 0, -1, -8])], x[t])
    with pytest.raises(IndexError, match="out of bounds"):
        kv_ops.block_index_tensor([0, 8], 8, cpu)
    with pytest.raises(IndexError, match="out of bounds"):
        kv_ops.block_index_tensor([-9], 8, cpu)
    assert kv_ops.block_index_tensor([], 8, cpu).numel() == 0
    assert kv_ops.block_index_tensor(np.array([1, 2]), 8, cpu).tolist() == [1, 2]
    with pytest.raises(TypeError):
        kv_ops.block_index_tensor(torch.tensor([1], dtype=torch.int32), 8, cpu)


def test_row_geometry_and_host_ids_short_paths():
    """The per-call checks have short paths (contiguous tensors, short lists); both paths give what the
    definitions say."""
    qkv = torch.zeros((7, 3 * 24))
    for x, want in ((torch.zeros((7, 4, 6)), (7, 24, 24)), (qkv[:, 24:48].view(7, 4, 6), (7, 24, 72)),
                    (torch.zeros((1, 4, 6)), (1, 24, 24)), (torch.zeros((0, 4, 6)), (0, 24, 24)),
                    (torch.zeros(5), (5, 1, 1)), (torch.zeros(10)[::2], (5, 1, 2)),
                    (torch.zeros((3, 1, 8)), (3, 8, 8))):
        assert kv_ops._row_geometry(x, "x") == want
    with pytest.raises(ValueError):
        kv_ops._row_geometry(torch.zeros((7, 6, 4)).transpose(1, 2), "x")  # rows not dense
    for ids in ([3, -1, 5], list(range(100)) + [-100], (2, 0), [[1, 2], [3, -4]], [], np.array([4, -2])):
        got = kv_ops.host_block_ids(ids, 100)
        want = np.asarray(ids, dtype=np.int64).reshape(-1)
        assert got.dtype == np.int64 and got.tolist() == np.where(want < 0, want + 100, want).tolist()
    for bad in ([3, 100], [-101], list(range(70)) + [100]):
        with pytest.raises(IndexError):
            kv_ops.host_block_ids(bad, 100)


def test_ops_refuse_cpu_tensors():
    pool = [torch.zeros((2, 4, 2, 1, 8), dtype=torch.float16)]
    with pytest.raises(RuntimeError, match="GPU only"):
        kv_ops.PoolView(pool)
    k = torch.zeros((2, 1, 8), dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU only"):
        kv_ops.reshape_and_cache(k, k, pool[0][0], pool[0][1], torch.tensor([0, 1]))
    # the layout variants and the vision gather refuse them too (no CPU fallback anywhere)
    kc = torch.zeros((4, 1, 1, 2, 8), dtype=torch.float16)
    vc = torch.zeros((4, 1, 8, 2), dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU only"):
        kv_ops.reshape_and_cache_paged(k, k, kc, vc, torch.tensor([0, 1]))
    with pytest.raises(RuntimeError, match="GPU only"):
        kv_ops.reshape_and_cache_strided([k], [k], [pool[0][0].permute(0, 2, 1, 3)], [pool[0][1].permute(0, 2, 1, 3)],
                                         torch.tensor([0, 1]))
    with pytest.raises(RuntimeError, match="GPU only"):
        kv_ops.concat_rows([k, k])
    with pytest.raises(RuntimeError, match="GPU only"):
        kv_ops.RowSource(k)


def test_worker_error_conventions_without_pool():
    w = KVWorker(device="cpu")
    with pytest.raises(RuntimeError, match="KV cache not initialized"):
        w.extract_kv_blocks([0])
    with pytest.raises(RuntimeError, match="KV cache not initialized"):
        w.write_kv_blocks([0], torch.zeros(1))
    assert w.get_kv_cache_layout() == {}
    assert w.p2p_send_kv(1, [0]) == {"error": "Global NCCL not initialized", "bytes": 0, "blocks": 0}
    assert w.p2p_recv_kv(1, [0]) == {"error": "Global NCCL not initialized", "bytes": 0, "blocks": 0}
    with pytest.raises(RuntimeError, match="NCCL not initialized"):
        w.p2p_coordinated_transfer_kv(None, 0, [1], [2])
    with pytest.raises(RuntimeError, match="NCCL not initialized"):
        w.p2p_pull_kv(0, [1], [2])
    assert w.get_global_rank() == -1 and w.init_global_nccl() is False
    with pytest.raises(RuntimeError, match="Vision embedding cache not initialized"):
        w.extract_vision_blocks("r")
    w.init_vecache()
    with pytest.raises(KeyError, match="not found in vision cache"):
        w.extract_vision_blocks("r")
    e = torch.zeros((3, 4))
    w.write_vision_blocks("r", e)
    assert w.extract_vision_blocks("r") is e
    assert w.gather_vision_embeddings(["r"]) is e
    assert w.gather_vision_embeddings(["missing"]) is None


def test_worker_shape_accessors_and_request_cleanup():
    w = KVWorker(device="cpu")
    assert w.get_kv_cache_shape() == () and w.get_ve_cache_shape() == ()
    assert w.get_ve_cache_keys() == [] and w.get_ve_shape("r") is None
    w.kv_cache = [torch.zeros((2, 5, 16, 4, 8)) for _ in range(3)]  # shape only: no kernel runs here
    assert w.get_kv_cache_shape() == (3, 2, 5, 16, 4, 8)
    w.init_vecache()
    w.write_vision_blocks("r", torch.zeros((3, 4)))
    w.write_vision_blocks("q", torch.zeros((7, 4)))
    assert w.get_ve_cache_keys() == ["r", "q"] and w.get_ve_shape("q") == (7, 4)
    w.swap_event_table.update({"r": object(), "q": object(), "z": object()})
    w.clear_request_resource_batched(["r", "q", "never seen"])
    assert list(w.swap_event_table) == ["z"]
    w.clear_all_requests()
    assert w.get_ve_cache_keys() == [] and w.swap_event_table == {} and w.ve_cache == {}


def test_migration_manager_registry_and_failures():
    import asyncio
    from elasticmm_amd.kv_transfer import KVMigrationManager

    class Fake:
        def __init__(self):
            self.blocks, self.ve = {}, {}

        def extract_kv_blocks(self, ids):
            return [self.blocks[i] for i in ids]  # KeyError for an unknown block

        def write_kv_blocks(self, ids, data):
            self.blocks.update(zip(ids, data))

        def extract_vision_blocks(self, rid):
            return self.ve[rid]

        def write_vision_blocks(self, rid, data):
            self.ve[rid] = data

    a, b = Fake(), Fake()
    a.blocks = {1: "x", 2: "y"}
    a.ve = {"r": "emb"}
    m = KVMigrationManager()
    assert asyncio.run(m.migrate_kv_blocks("r", "prefill", 0, [1], "decoding", 0, [5])) is False
    m.register_worker("PREFILL", 0, a)
    m.register_worker("decoding", 0, b)
    assert asyncio.run(m.migrate_kv_blocks("r", "prefill", 0, [2, 1], "decoding", 0, [5, 6])) is True
    assert b.blocks == {5: "y", 6: "x"}
    assert asyncio.run(m.migrate_vision_embeddings("r", "prefill", 0, "decoding", 0)) is True and b.ve == {"r": "emb"}
    assert m.migrate_kv_blocks_sync("r", "prefill", 0, [9], "decoding", 0, [5]) is False
    assert m.migrate_vision_embeddings_sync("nope", "prefill", 0, "decoding", 0) is False
    st = m.get_stats()
    assert st["migration_count"] == 2 and st["avg_migration_time"] >= 0.0
    assert KVMigrationManager().get_stats()["avg_migration_time"] == 0.0


def test_coordinated_transfer_preflight():
    link = LoopbackLink(world_size=2)
    w = KVWorker(device="cpu", link=link, global_rank=1)
    with pytest.raises(ValueError, match="Block count mismatch: src=2, dst=1"):
        w.p2p_coordinated_transfer_kv(None, 0, [1, 2], [3])
    assert w.p2p_coordinated_transfer_kv(None, 0, [], []) == {"bytes": 0, "blocks": 0, "error": "No blocks to transfer"}
    with pytest.raises(ValueError, match="Invalid src_rank"):
        w.p2p_coordinated_transfer_kv(None, 5, [1], [2])
    with pytest.raises(ValueError, match="Unsupported dtype"):
        w.collective_transfer_kv("g", 0, [0], (1,), "float8_e4m3fn", "send")


def test_loopback_link_fifo():
    link = LoopbackLink(2)
    a, b = torch.zeros(1), torch.ones(1)
    link.send(a, 0, 1)
    link.send(b, 0, 1)
    assert link.pending(0, 1) == 2
    assert link.recv(0, 1) is a and link.recv(0, 1) is b
    with pytest.raises(RuntimeError, match="no message pending"):
        link.recv(0, 1)
    with pytest.raises(ValueError, match="Invalid dst rank"):
        link.send(a, 0, 7)


def test_block_manager_free_list_order():
    bm = BlockManager(8, block_size=16)
    assert bm.get_num_blocks_needed(17) == 2
    assert bm.allocate_blocks("a", 3) == [0, 1, 2]
    assert bm.allocate_blocks("b", 2) == [3, 4]
    bm.free_blocks("a")
    assert bm.allocate_blocks("c", 4) == [5, 6, 7, 0]  # freed blocks rejoin at the end
    assert bm.allocate_blocks("b", 3) == [3, 4, 1]      # growth appends
    assert bm.get_block_table("zz") == []
    with pytest.raises(AssertionError, match="Not enough free blocks"):
        bm.allocate_blocks("d", 5)
    ids = bm.get_block_table("b") + bm.get_block_table("c")
    assert len(set(ids)) == len(ids)


class _Req:
    def __init__(self, request_id, total_len, images=None):
        self.request_id, self.total_len, self.images = request_id, total_len, images

    def get_total_len(self):
        return self.total_len


class _SwapRecorder:
    def __init__(self):
        self.calls = []

    def swap_blocks(self, request_ids, src, dst, is_swap_in):
        self.calls.append(("swap_blocks", list(request_ids), list(src), list(dst), is_swap_in))

    def wait_for_all_swap_in(self):
        self.calls.append(("wait_in",))

    def wait_for_all_swap_out(self):
        self.calls.append(("wait_out",))

    def clear_request_resource(self, request_id):
        self.calls.append(("clear", request_id))


def test_block_manager_requests_growth_and_queries():
    bm = BlockManager(10, block_size=16, max_num_cpu_blocks=4)
    a, b = _Req("a", 33), _Req("b", 16)
    assert bm.get_num_blocks_needed(a) == 3 and bm.can_allocate(a)
    assert bm.allocate_blocks(a) == [0, 1, 2]
    bm.allocate_blocks_batched([b])
    assert bm.get_block_table("b") == [3] and bm.get_location("b") == BlockLocation.GPU
    a.total_len = 49                       # one decode step past a block boundary
    assert bm.get_num_append_blocks_needed(a) == 1 and bm.can_append(a)
    bm.append_blocks(a)
    assert bm.get_block_table("a") == [0, 1, 2, 4]
    bm.append_blocks(a)                    # nothing to add
    assert bm.get_allocated_num_blocks("a") == 4
    assert bm.expand_blocks_for_seq_len("b", 40) == [3, 5, 6]      # vision tokens spliced in
    assert bm.expand_blocks_for_seq_len("b", 8) == [3, 5, 6]
    with pytest.raises(ValueError, match="not allocated"):
        bm.expand_blocks_for_seq_len("zz", 8)
    with pytest.raises(ValueError, match="explicit num_blocks"):
        bm.allocate_blocks("plain-id")
    assert bm.get_max_blocks_needed([a, b, _Req("c", 100)]) == 7
    assert not bm.can_allocate(_Req("c", 100)) and bm.can_append(_Req("d", 48))
    assert bm.get_block_usage() == {"gpu": "70% (7/10)", "cpu": "0% (0/4)", "swap": "0 -> 0", "#req": "2"}
    bm.free_blocks_batched([a, "b", "unknown"])
    assert bm.get_num_avail_gpu_blocks() == 10 and bm.free_gpu_blocks_list[-7:] == [0, 1, 2, 4, 3, 5, 6]
    vb = VisionBlockManager(100, block_size=16)
    assert vb.get_num_blocks_needed(_Req("v", 5, images=["i0", "i1"])) == 72 and vb.get_num_blocks_needed(_Req("t", 5)) == 0


def test_block_manager_pool_tensors_for_a_batch(capsys):
    from types import SimpleNamespace as NS

    bm = BlockManager(64, block_size=16, max_num_cpu_blocks=8, stage="decoding")
    batch = NS(requests=[40, 17, 100])  # token counts stand for requests
    assert bm.get_max_blocks_needed(batch) == 7 and bm.get_max_blocks_needed([1]) == 1
    layers = bm.create_kv_cache_tensors(batch, num_layers=3, num_heads=2, head_size=8, dtype=torch.float16, device="cpu")
    assert len(layers) == 3 and all(t.shape == (2, 7, 16, 2, 8) and t.dtype == torch.float16 for t in layers)
    assert bm.create_kv_cache_tensors([], 2, 1, 8, torch.float16, "cpu")[0].shape == (2, 0, 16, 1, 8)
    bm.allocate_blocks("a", 16)
    bm.print_block_usage()
    assert capsys.readouterr().out.strip() == "(decoding) Block usage: GPU=25% (16/64), CPU=0% (0/8), Swapping=0 -> 0, Requests=1"


def test_block_manager_conserves_blocks_under_random_operations():
    """2000 seeded random operations (allocate, grow, free, swap out, swap in, with a worker that records the
    copies it is asked for): after every one of them each GPU block id and each CPU block id is in exactly one
    place: a request's table, the free list, or the list of blocks whose copy is still in flight."""
    import random

    class Recorder:
        def __init__(self):
            self.copies = 0

        def swap_blocks(self, request_ids, src, dst, is_swap_in):
            assert len(src) == len(dst) and len(set(dst)) == len(dst)
            self.copies += len(src)

        def wait_for_all_swap_in(self):
            pass

        def wait_for_all_swap_out(self):
            pass

        def clear_request_resource(self, request_id):
            pass

    rng = random.Random(1234)
    G, C = 48, 32
    rec = Recorder()
    bm = BlockManager(G, block_size=16, max_num_cpu_blocks=C, workers=[rec])
    live, next_id = [], 0

    def check():
        gpu = list(bm.free_gpu_blocks_list) + list(bm.swapping_gpu_blocks_list)
        cpu = list(bm.free_cpu_blocks_list) + list(bm.swapping_cpu_blocks_list)
        for rid, table in bm.block_table.items():
            (gpu if bm.get_location(rid) == BlockLocation.GPU else cpu).extend(table)
        assert sorted(gpu) == list(range(G)) and sorted(cpu) == list(range(C))
        assert set(bm.block_table) == set(live) == set(bm.request_location)

    for _ in range(2000):
        op = rng.choice(["alloc", "alloc", "grow", "free", "out", "in"])
        on_gpu = [r for r in live if bm.get_location(r) == BlockLocation.GPU]
        on_cpu = [r for r in live if bm.get_location(r) == BlockLocation.CPU]
        if op == "alloc":
            n = rng.randint(1, 9)
            if bm.get_num_avail_gpu_blocks() >= n:
                rid = f"r{next_id}"
                next_id += 1
                assert len(bm.allocate_blocks(rid, n)) == n
                live.append(rid)
        elif op == "grow" and on_gpu:
            rid = rng.choice(on_gpu)
            want = bm.get_allocated_num_blocks(rid) + rng.randint(0, 3)
            if bm.get_num_avail_gpu_blocks() >= want - bm.get_allocated_num_blocks(rid):
                assert len(bm.expand_blocks_for_seq_len(rid, want * 16)) == want
        elif op == "free" and live:
            rid = rng.choice(live)
            bm.free_blocks(rid)
            live.remove(rid)
        elif op == "out" and on_gpu:
            rids = rng.sample(on_gpu, min(len(on_gpu), rng.randint(1, 3)))
            if bm.get_num_avail_cpu_blocks() >= sum(bm.get_allocated_num_blocks(r) for r in rids):
                bm.swap_out_requests(rids)
        elif op == "in" and on_cpu:
            rids = rng.sample(on_cpu, min(len(on_cpu), rng.randint(1, 3)))
            if bm.get_num_avail_gpu_blocks() >= sum(bm.get_allocated_num_blocks(r) for r in rids):
                bm.swap_in_requests(rids)
        check()
    assert rec.copies > 100 and next_id > 100


def test_block_manager_swap_bookkeeping_and_worker_calls():
    rec = _SwapRecorder()
    bm = BlockManager(6, block_size=16, max_num_cpu_blocks=5, workers=[rec])
    bm.allocate_blocks("r1", 2)
    bm.allocate_blocks("r2", 3)
    src, dst = bm.swap_out_requests(["r1", "r2"])
    assert (src, dst) == ([0, 1, 2, 3, 4], [0, 1, 2, 3, 4])
    assert rec.calls == [("swap_blocks", ["r1", "r2"], [0, 1, 2, 3, 4], [0, 1, 2, 3, 4], False)]
    assert bm.get_location("r1") == BlockLocation.CPU and not bm.is_all_requests_on_gpu(["r1"])
    assert bm.get_block_table("r2") == [2, 3, 4]
    # the GPU blocks being copied out count as available but are only handed out after the workers were waited for
    assert bm.get_num_avail_gpu_blocks() == 6 and bm.free_gpu_blocks_list == [5]
    assert bm.get_block_usage()["swap"] == "5 -> 0"
    assert bm.allocate_blocks("r3", 1) == [5] and rec.calls[-1][0] == "swap_blocks"
    assert bm.allocate_blocks("r4", 2) == [0, 1] and rec.calls[-1] == ("wait_out",)
    with pytest.raises(AssertionError, match="is on CPU"):
        bm.allocate_blocks("r1", 3)
    with pytest.raises(AssertionError, match="is on BlockLocation.CPU now"):
        bm.swap_out_requests(["r1"])
    src, dst = bm.swap_in_requests(["r2"])
    assert (src, dst) == ([2, 3, 4], [2, 3, 4]) and rec.calls[-1] == ("swap_blocks", ["r2"], [2, 3, 4], [2, 3, 4], True)
    assert bm.free_cpu_blocks_list == [] and bm.swapping_cpu_blocks_list == [2, 3, 4]
    # CPU blocks parked by the swap-in are reused only after wait_for_all_swap_in
    bm.swap_out_requests(["r3"])
    assert rec.calls[-2] == ("wait_in",) and bm.get_block_table("r3") == [2]
    with pytest.raises(AssertionError, match="Not enough free blocks on CPU"):
        bm.swap_out_requests(["r2", "r4"])
    bm.clear_request_resource_batched(["r1", "r2"])
    assert rec.calls[-2:] == [("clear", "r1"), ("clear", "r2")]
    bm.free_blocks("r1")
    assert bm.free_cpu_blocks_list[-2:] == [0, 1] and bm.swap_count == 3
    calls = []
    bm2 = BlockManager(2, max_num_cpu_blocks=2, engine_remote_call_all_workers_async=lambda *a: calls.append(a))
    bm2.allocate_blocks("x", 2)
    bm2.swap_out_requests(["x"])
    assert calls == [("swap_blocks", ["x"], [0, 1], [0, 1], False)]


# ------------------------------------------------------------------ transfer manager (fake workers)
class _FakeWorker:
    def __init__(self, rank, fail=False):
        self.rank, self.fail, self.calls = rank, fail, []

    def extract_kv_blocks(self, blocks):
        self.calls.append(("extract", list(blocks)))
        return ("data", list(blocks))

    def write_kv_blocks(self, blocks, data):
        self.calls.append(("write", list(blocks), data))

    def p2p_coordinated_transfer_kv(self, src, src_rank, src_blocks, dst_blocks, timeout=10.0):
        self.calls.append(("coord", src_rank, list(src_blocks), list(dst_blocks), timeout))
        if self.fail:
            return {"error": "boom", "bytes": 0, "blocks": 0}
        return {"bytes": 100 * len(dst_blocks), "blocks": len(dst_blocks)}

    def p2p_send_kv(self, dst_rank, blocks):
        self.calls.append(("send", dst_rank, list(blocks)))
        return {"bytes": 100 * len(blocks), "blocks": len(blocks)}

    def p2p_recv_kv(self, src_rank, blocks):
        self.calls.append(("recv", src_rank, list(blocks)))
        return {"bytes": 100 * len(blocks), "blocks": len(blocks)}


def test_transfer_manager_dispatch_stats_and_batching():
    import asyncio

    from elasticmm_amd.kv_transfer import KVTransferManager, TransferMethod

    seen = []
    m = KVTransferManager(TransferMethod.NCCL, metrics_callback=lambda **kw: seen.append(kw))
    a, b = _FakeWorker(0), _FakeWorker(1)
    m.register_workers("Prefill", [a, None], [0, -1])
    m.register_worker(1, b, "DECODING")
    assert m.rank_to_stage == {0: "prefill", 1: "decoding"}
    assert asyncio.run(m.transfer_kv_cache("r0", 0, 1, [1, 2], [7, 8])) is True
    assert b.calls[-1] == ("coord", 0, [1, 2], [7, 8], 10.0)
    # the first transfer is the cold start: counted by the callback, not by the statistics
    assert m.get_stats()["transfer_count"] == 0 and len(seen) == 1 and seen[0]["num_blocks"] == 2
    assert m.transfer_kv_cache_sync("r1", 0, 1, [3], [9]) is True
    st = m.get_stats()
    assert st["transfer_count"] == 1 and st["total_bytes_transferred"] == 100 and st["avg_transfer_time"] >= 0.0
    assert m.transfer_kv_cache_sync("r2", 0, 5, [3], [9]) is False            # unknown rank
    b.fail = True
    assert m.transfer_kv_cache_sync("r3", 0, 1, [3], [9]) is False            # error dict -> False
    m.reset_stats()
    assert m.get_stats()["transfer_count"] == 0
    m.update_worker_stage(1, "Prefill")
    assert m.rank_to_stage[1] == "prefill"
    m.unregister_worker(1)
    assert 1 not in m.worker_registry

    # p2p_copy: extract on the source, write on the destination
    m2 = KVTransferManager(TransferMethod.P2P_COPY)
    a, b = _FakeWorker(0), _FakeWorker(1)
    m2.register_workers("prefill", [a, b], [0, 1])
    assert m2.transfer_kv_cache_sync("r", 0, 1, [4, 5], [6, 7]) is True
    assert a.calls == [("extract", [4, 5])] and b.calls == [("write", [6, 7], ("data", [4, 5]))]
    assert m2.get_stats()["transfer_count"] == 1
    assert KVTransferManager(TransferMethod.STAGED_COPY).transfer_kv_cache_sync("r", 0, 1, [1], [2]) is False

    # batching: three requests are merged into one send / one recv with concatenated tables
    m3 = KVTransferManager(TransferMethod.NCCL, enable_batching=True, batch_size=3, batch_timeout=1e9)
    a, b = _FakeWorker(0), _FakeWorker(1)
    m3.register_workers("prefill", [a, b], [0, 1])
    assert m3.transfer_kv_cache_sync("q0", 0, 1, [1, 2], [11, 12]) is True and not a.calls
    assert m3.transfer_kv_cache_sync("q1", 0, 1, [3], [13]) is True and not a.calls
    assert m3.transfer_kv_cache_sync("q2", 0, 1, [4, 5], [14, 15]) is True
    assert a.calls == [("send", 1, [1, 2, 3, 4, 5])] and b.calls == [("recv", 0, [11, 12, 13, 14, 15])]
    assert m3.get_stats()["transfer_count"] == 3 and m3.get_stats()["total_bytes_transferred"] == 500
    assert m3.transfer_kv_cache_sync("q3", 0, 1, [6], [16]) is True and len(a.calls) == 1
    assert m3.flush_all() is True and a.calls[-1] == ("send", 1, [6])


def test_migrate_requests_allocates_moves_frees_and_rolls_back():
    src_bm, dst_bm = BlockManager(16), BlockManager(6)
    src_bm.allocate_blocks("a", 3)
    src_bm.allocate_blocks("b", 2)
    src_bm.allocate_blocks("big", 5)
    tm = KVTransferManager(TransferMethod.P2P_COPY)
    w0, w1 = _FakeWorker(0), _FakeWorker(1)
    tm.register_worker(0, w0, "prefill")
    tm.register_worker(1, w1, "decoding")
    assert tm.migrate_requests_sync(["a", "none", "b"], 0, src_bm, 1, dst_bm)
    assert w0.calls == [("extract", [0, 1, 2]), ("extract", [3, 4])]
    assert [c[:2] for c in w1.calls] == [("write", [0, 1, 2]), ("write", [3, 4])]
    assert src_bm.get_block_table("a") == [] and dst_bm.get_block_table("b") == [3, 4]
    assert src_bm.free_gpu_blocks_list[-5:] == [0, 1, 2, 3, 4]
    # the destination cannot hold the request: nothing moves, nothing leaks
    assert not tm.migrate_requests_sync(["big"], 0, src_bm, 1, dst_bm)
    assert src_bm.get_block_table("big") == [5, 6, 7, 8, 9] and dst_bm.get_num_avail_gpu_blocks() == 1
    # a failing transfer after a successful one: the destination is rolled back, the source keeps everything
    dst_bm.free_blocks("a")
    src_bm.allocate_blocks("c", 1)
    src_bm.allocate_blocks("e", 1)
    tm.unregister_worker(1)
    bad = _FakeWorker(1)
    bad.write_kv_blocks = lambda blocks, data: (_ for _ in ()).throw(RuntimeError("link down")) if len(bad.calls) else bad.calls.append("first")
    tm.register_worker(1, bad, "decoding")
    assert not tm.migrate_requests_sync(["c", "e"], 0, src_bm, 1, dst_bm)
    assert dst_bm.get_block_table("c") == [] and dst_bm.get_block_table("e") == []
    assert src_bm.get_block_table("c") != [] and src_bm.get_block_table("e") != []


def test_batched_migration_rollback_leaves_nothing_queued():
    """With batching, requests that were already queued when a later allocation fails must leave the queue
    before their destination blocks are freed: a later flush may not touch the destination."""
    src_bm, dst_bm = BlockManager(16), BlockManager(4)
    src_bm.allocate_blocks("a", 2)
    src_bm.allocate_blocks("b", 1)
    src_bm.allocate_blocks("c", 3)          # does not fit once a and b hold 3 of the 4 destination blocks
    tm = KVTransferManager(TransferMethod.NCCL, enable_batching=True, batch_size=10, batch_timeout=1e9)
    w0, w1 = _FakeWorker(0), _FakeWorker(1)
    tm.register_worker(0, w0, "prefill")
    tm.register_worker(1, w1, "decoding")
    assert not tm.migrate_requests_sync(["a", "b", "c"], 0, src_bm, 1, dst_bm)
    assert tm._transfer_queue.get((0, 1), []) == []
    assert tm.flush_all() is True
    assert w0.calls == [] and w1.calls == []                  # nothing was sent, nothing was written
    assert dst_bm.get_num_avail_gpu_blocks() == 4             # destination blocks all free again
    assert src_bm.get_block_table("a") == [0, 1] and src_bm.get_block_table("c") == [3, 4, 5]
    # an unrelated request queued before the failing migration stays queued and is flushed normally
    assert tm.transfer_kv_cache_sync("other", 0, 1, [9], [3]) is True
    assert not tm.migrate_requests_sync(["a", "b", "c"], 0, src_bm, 1, dst_bm)
    assert [t[0] for t in tm._transfer_queue[(0, 1)]] == ["other"]
    assert tm.flush_all() is True and w0.calls == [("send", 1, [9])] and w1.calls == [("recv", 0, [3])]


def test_concurrent_coroutines_keep_block_tables_disjoint_and_run_on_the_calling_thread():
    """Two migrations and a scheduler that allocates from the same destination block manager, all in flight
    on one event loop: a transfer has no await point inside, so its bookkeeping is atomic with respect to the
    other coroutines — no block id is ever handed out twice — and it runs on the calling thread (where torch's
    current stream is the caller's)."""
    import asyncio
    import threading

    from elasticmm_amd.block_manager import BlockManager

    loop_thread = threading.get_ident()
    threads = set()

    class _W(_FakeWorker):
        def extract_kv_blocks(self, blocks):
            threads.add(threading.get_ident())
            return super().extract_kv_blocks(blocks)

    tm = KVTransferManager(TransferMethod.P2P_COPY)
    tm.register_worker(0, _W(0), "prefill")
    tm.register_worker(1, _W(1), "decoding")
    src_bm, dst_bm = BlockManager(64), BlockManager(64)
    for i in range(8):
        src_bm.allocate_blocks(f"r{i}", 3)
    taken = {}

    async def scheduler():
        for i in range(10):
            dst_bm.allocate_blocks(f"s{i}", 2)
            taken[f"s{i}"] = list(dst_bm.get_block_table(f"s{i}"))
            await asyncio.sleep(0)

    async def main():
        return await asyncio.gather(tm.migrate_requests([f"r{i}" for i in range(4)], 0, src_bm, 1, dst_bm), scheduler(),
                                    tm.migrate_requests([f"r{i}" for i in range(4, 8)], 0, src_bm, 1, dst_bm))

    ok1, _, ok2 = asyncio.run(main())
    assert ok1 is True and ok2 is True and threads == {loop_thread}
    tables = [dst_bm.get_block_table(f"r{i}") for i in range(8)] + list(taken.values())
    flat = [b for t in tables for b in t]
    assert len(flat) == 8 * 3 + 10 * 2 and len(set(flat)) == len(flat), "a block id was handed out twice"
    assert all(src_bm.get_block_table(f"r{i}") in (None, []) for i in range(8))   # the source blocks were freed
    tm.close()


def test_two_managers_share_one_link_without_mixing_their_transfers():
    """A KVTransferManager (NCCL method, batched) and a KVMigrationManager working over the same two workers and
    the same link: the layers of one transfer are never interleaved with another's, and a failed receive drops
    only its own transfer's messages."""
    import asyncio

    from elasticmm_amd.kv_transfer import KVMigrationManager
    from elasticmm_amd.worker import LoopbackLink

    link = LoopbackLink(2)

    class _LinkWorker:
        """The link protocol of KVWorker.p2p_send_kv / p2p_recv_kv (three layer messages per transfer) on plain lists."""
        def __init__(self, rank):
            self.rank, self.link, self.store, self.fail_recv = rank, link, {}, False

        def p2p_send_kv(self, dst_rank, blocks):
            tid = self.link.new_transfer_id()
            for l in range(3):
                self.link.send([(l, b, self.store.get(b)) for b in blocks], src=self.rank, dst=dst_rank, transfer_id=tid)
            self.last_sent_transfer_id = tid
            return {"bytes": 3 * len(blocks), "blocks": len(blocks)}

        def p2p_recv_kv(self, src_rank, blocks):
            if self.fail_recv:
                return {"error": "refused", "bytes": 0, "blocks": 0}
            tid = self.link.head_id(src_rank, self.rank)
            for l in range(3):
                got_tid, msg = self.link.recv_with_id(src_rank, self.rank)
                assert got_tid == tid and [m[0] for m in msg] == [l] * len(blocks), "layers of two transfers interleaved"
                for (_, _, val), b in zip(msg, blocks):
                    self.store[b] = val
            return {"bytes": 3 * len(blocks), "blocks": len(blocks)}

        def extract_kv_blocks(self, blocks):
            return [self.store[b] for b in blocks]

        def write_kv_blocks(self, blocks, data):
            self.store.update(zip(blocks, data))

    a, b = _LinkWorker(0), _LinkWorker(1)
    a.store = {i: f"v{i}" for i in range(10)}
    tm = KVTransferManager(TransferMethod.NCCL, enable_batching=True, batch_size=2, batch_timeout=1e9)
    tm.register_worker(0, a, "prefill")
    tm.register_worker(1, b, "decoding")
    mm = KVMigrationManager()
    mm.register_worker("prefill", 0, a)
    mm.register_worker("decoding", 0, b)

    async def main():
        return await asyncio.gather(tm.transfer_kv_cache("x", 0, 1, [0, 1], [20, 21]),
                                    mm.migrate_kv_blocks("m", "prefill", 0, [2], "decoding", 0, [22]),
                                    tm.transfer_kv_cache("y", 0, 1, [3], [23]),        # second of the batch: flushes
                                    mm.migrate_kv_blocks("n", "prefill", 0, [4], "decoding", 0, [24]))

    assert asyncio.run(main()) == [True, True, True, True]
    assert {k: b.store[k] for k in (20, 21, 22, 23, 24)} == {20: "v0", 21: "v1", 22: "v2", 23: "v3", 24: "v4"}
    assert link.pending(0, 1) == 0
    # a receive that refuses: only that transfer's three messages leave the link; a transfer queued earlier by
    # somebody else between the same ranks stays
    other = link.new_transfer_id()
    link.send(["somebody else's layer"], src=0, dst=1, transfer_id=other)
    b.fail_recv = True
    assert tm.transfer_kv_cache_sync("z", 0, 1, [5], [25]) is True                      # queued
    assert tm.transfer_kv_cache_sync("w", 0, 1, [6], [26]) is False                     # flush: receive refused
    assert link.pending(0, 1) == 1 and link.head_id(0, 1) == other


def test_vision_transfer_through_the_manager_with_fake_workers():
    class _VeWorker(_FakeWorker):
        def __init__(self, rank):
            super().__init__(rank)
            self.ve = {}

        def extract_vision_blocks(self, rid):
            if rid not in self.ve:
                raise KeyError(f"Request {rid} not found in vision cache")
            return self.ve[rid]

        def write_vision_blocks(self, rid, data):
            self.ve[rid] = data

    seen = []
    tm = KVTransferManager(TransferMethod.NCCL, metrics_callback=lambda **kw: seen.append(kw))
    a, b = _VeWorker(0), _VeWorker(1)
    a.ve["img"] = "embedding"
    tm.register_workers("encoding", [a, b], [0, 1])
    assert tm.transfer_vision_embeddings_sync("img", 0, [1], 1, [2]) is True and b.ve["img"] == "embedding"
    assert tm.transfer_vision_embeddings_sync("none", 0, [], 1, []) is False
    assert tm.transfer_vision_embeddings_sync("img", 0, [1], 7, [2]) is False      # unknown rank
    assert tm.get_stats()["transfer_count"] == 1 and seen == []                     # counted, not a kv metric


def test_compute_slot_mapping_matches_the_definition():
    from elasticmm_amd import cache_ops

    tables = [[7, 2, 9], [4], [5, 0]]
    ctx, q, bs = [0, 3, 17], [40, 1, 2], 16
    got = cache_ops.compute_slot_mapping(tables, ctx, q, bs, pad_to=48)
    want = []
    for t, c, n in zip(tables, ctx, q):
        for p in range(c, c + n):
            want.append(t[p // bs] * bs + p % bs)
    assert got.dtype == torch.long and got.tolist() == want + [-1] * 5
    assert got[:16].tolist() == list(range(7 * 16, 8 * 16))          # a prompt fills its blocks in order
    assert cache_ops.compute_slot_mapping([], [], [], 16).numel() == 0
    assert cache_ops.compute_slot_mapping([[1]], [0], [0], 16, pad_to=3).tolist() == [-1, -1, -1]
    with pytest.raises(IndexError, match="needs 3 blocks"):
        cache_ops.compute_slot_mapping([[1, 2]], [0], [33], 16)
    with pytest.raises(ValueError, match="pad_to"):
        cache_ops.compute_slot_mapping([[1, 2]], [0], [20], 16, pad_to=8)
    with pytest.raises(ValueError, match="differ in length"):
        cache_ops.compute_slot_mapping([[1]], [0, 1], [1], 16)
