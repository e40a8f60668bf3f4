"""Host-side logic of the drop-in surface (no GPU needed)."""
import numpy as np
import pytest
import torch

from elasticmm_amd import kv_ops
from elasticmm_amd.block_manager import BlockManager
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


def test_ops_refuse_cpu_tensors():
    pool = [torch.zeros((2, 4, 2, 1, 8), dtype=torch.float16)]
    with pytest.raises(RuntimeError, match="GPU only"):
        kv_ops.PoolView(pool)
    k = torch.zeros((2, 1, 8), dtype=torch.float16)
    with pytest.raises(RuntimeError, match="GPU only"):
        kv_ops.reshape_and_cache(k, k, pool[0][0], pool[0][1], torch.tensor([0, 1]))


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
