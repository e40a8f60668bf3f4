"""Host-side block tables: the index producer of the KV path.

A free-list allocator with the observable behaviour of the reference's
``V0BlockManager`` (elasticmm/engine/v0/block_manager.py:102-142, :174-209,
:264-266): blocks are handed out from the front of the free list, freed blocks
are appended to its end, so a request's table is a list of unique Python ints in
arbitrary order. Swap bookkeeping and the CPU tier are not part of this path.
"""
from __future__ import annotations

from typing import Dict, List


class BlockManager:
    def __init__(self, max_num_gpu_blocks: int, block_size: int = 16):
        self.max_num_gpu_blocks = max_num_gpu_blocks
        self.block_size = block_size
        self.free_gpu_blocks_list: List[int] = list(range(max_num_gpu_blocks))
        self.block_table: Dict[str, List[int]] = {}

    def get_num_avail_gpu_blocks(self) -> int:
        return len(self.free_gpu_blocks_list)

    def get_num_blocks_needed(self, num_tokens: int) -> int:
        return (num_tokens + self.block_size - 1) // self.block_size

    def _get_free_blocks(self, num_blocks: int) -> List[int]:
        num_avail_blocks = self.get_num_avail_gpu_blocks()
        assert num_avail_blocks >= num_blocks, \
            f"Not enough free blocks on GPU, requested {num_blocks}, available {num_avail_blocks}"
        blocks = self.free_gpu_blocks_list[:num_blocks]
        self.free_gpu_blocks_list = self.free_gpu_blocks_list[num_blocks:]
        return blocks

    def allocate_blocks(self, request_id: str, num_blocks: int) -> List[int]:
        """First allocation takes ``num_blocks``; later calls grow the table up to it."""
        if request_id not in self.block_table:
            self.block_table[request_id] = self._get_free_blocks(num_blocks)
        else:
            cur = len(self.block_table[request_id])
            if cur < num_blocks:
                self.block_table[request_id] += self._get_free_blocks(num_blocks - cur)
        return self.block_table[request_id]

    def free_blocks(self, request_id: str) -> None:
        assert request_id in self.block_table, f"Request {request_id} not allocated"
        self.free_gpu_blocks_list += self.block_table.pop(request_id)

    def get_block_table(self, request_id: str) -> List[int]:
        return self.block_table.get(request_id, [])
