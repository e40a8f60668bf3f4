"""Host-side block tables: the index producer of the KV path, with the GPU / CPU tiers.

Observable behaviour of the reference's ``V0BlockManager``
(elasticmm/engine/v0/block_manager.py): blocks are handed out from the front of a tier's free
list and freed blocks rejoin at its end (:102-142, :247-256), so a request's table is a list of
unique Python ints in arbitrary order; a table grows by appending (:174-209, :216-245, :281-300);
swapping a request moves its table to the other tier, parks the old blocks on a "swapping" list
that only becomes allocatable after the workers have been waited for, and hands the workers one
concatenated (source ids, target ids) pair per call (:305-377).

What is different: a request is anything with ``request_id`` and ``get_total_len()`` (or a plain
id string together with an explicit block count), and the worker call goes to ``KVWorker`` objects
in this process through ``workers=[...]`` (or to any callable with the reference's
``engine_remote_call_all_workers_async(name, *args)`` shape). Scheduling decisions are not made
here.
"""
from __future__ import annotations

from enum import Enum
from typing import Any, Callable, Dict, Iterable, List, Optional, Sequence, Tuple, Union


class BlockLocation(Enum):
    """block_manager.py:15-18."""
    GPU = "gpu"
    CPU = "cpu"


RequestLike = Union[str, Any]


def _request_id(request: RequestLike) -> str:
    return request if isinstance(request, str) else request.request_id


class BlockManager:
    def __init__(self, max_num_gpu_blocks: int, block_size: int = 16, max_num_cpu_blocks: int = 0,
                 stage: str = "prefill", workers: Optional[Sequence[Any]] = None,
                 engine_remote_call_all_workers_async: Optional[Callable[..., Any]] = None):
        self.stage = stage
        self.max_num_gpu_blocks = max_num_gpu_blocks
        self.max_num_cpu_blocks = max_num_cpu_blocks
        self.block_size = block_size
        self.workers = list(workers) if workers is not None else []
        self._remote_call = engine_remote_call_all_workers_async
        self.block_table: Dict[str, List[int]] = {}
        self.request_location: Dict[str, BlockLocation] = {}
        self.swap_count = 0
        self._reset_free_blocks()

    # ----- worker calls ---------------------------------------------------------
    def _call_workers(self, name: str, *args) -> None:
        if self._remote_call is not None:
            self._remote_call(name, *args)
        for w in self.workers:
            getattr(w, name)(*args)

    # ----- free lists (block_manager.py:75-142) ----------------------------------
    def _reset_free_blocks(self) -> None:
        self.free_gpu_blocks_list: List[int] = list(range(self.max_num_gpu_blocks))
        self.free_cpu_blocks_list: List[int] = list(range(self.max_num_cpu_blocks))
        self.swapping_gpu_blocks_list: List[int] = []
        self.swapping_cpu_blocks_list: List[int] = []

    def get_num_avail_gpu_blocks(self) -> int:
        return len(self.free_gpu_blocks_list) + len(self.swapping_gpu_blocks_list)

    def get_num_avail_cpu_blocks(self) -> int:
        return len(self.free_cpu_blocks_list) + len(self.swapping_cpu_blocks_list)

    def _get_free_blocks(self, num_blocks: int, location: BlockLocation = BlockLocation.GPU) -> List[int]:
        on_gpu = location == BlockLocation.GPU
        avail = self.get_num_avail_gpu_blocks() if on_gpu else self.get_num_avail_cpu_blocks()
        assert avail >= num_blocks, \
            f"Not enough free blocks on {'GPU' if on_gpu else 'CPU'}, requested {num_blocks}, available {avail}"
        free = self.free_gpu_blocks_list if on_gpu else self.free_cpu_blocks_list
        if len(free) < num_blocks:
            # blocks still being copied out of this tier become free once the copies are done
            self._call_workers("wait_for_all_swap_out" if on_gpu else "wait_for_all_swap_in")
            parked = self.swapping_gpu_blocks_list if on_gpu else self.swapping_cpu_blocks_list
            free += parked
            parked.clear()
        blocks = free[:num_blocks]
        del free[:num_blocks]
        return blocks

    # ----- queries -----------------------------------------------------------------
    def get_allocated_num_blocks(self, request_id: str) -> int:
        return len(self.block_table.get(request_id, []))

    def get_location(self, request_id: str) -> Optional[BlockLocation]:
        return self.request_location.get(request_id)

    def get_block_table(self, request_id: str) -> List[int]:
        return self.block_table.get(request_id, [])

    def get_num_blocks_needed(self, request: Union[int, Any]) -> int:
        """Blocks for a token count, or for ``request.get_total_len()`` (block_manager.py:152-163)."""
        total_len = request if isinstance(request, int) else request.get_total_len()
        return (total_len + self.block_size - 1) // self.block_size

    def get_num_append_blocks_needed(self, request: Any) -> int:
        rid = _request_id(request)
        assert self.request_location.get(rid) == BlockLocation.GPU, f"Request {rid} is not on GPU"
        return max(0, self.get_num_blocks_needed(request) - len(self.block_table[rid]))

    def get_max_blocks_needed(self, requests: Any) -> int:
        """block_manager.py:487-501; takes a BatchedRequests-like object (``.requests``) or an iterable."""
        requests = getattr(requests, "requests", requests)
        return max((self.get_num_blocks_needed(r) for r in requests), default=0)

    def can_allocate(self, request: Any) -> bool:
        return self.get_num_avail_gpu_blocks() >= self.get_num_blocks_needed(request)

    def can_append(self, request: Any) -> bool:
        if _request_id(request) not in self.block_table:
            return self.can_allocate(request)
        return self.get_num_avail_gpu_blocks() >= self.get_num_append_blocks_needed(request)

    def is_all_requests_on_gpu(self, request_ids: Iterable[str]) -> bool:
        return all(self.request_location.get(r) != BlockLocation.CPU for r in request_ids)

    # ----- allocation (block_manager.py:174-300) ---------------------------------------
    def allocate_blocks(self, request: RequestLike, num_blocks: Optional[int] = None) -> List[int]:
        """First allocation takes the blocks needed; later calls grow the table up to that count."""
        rid = _request_id(request)
        assert rid not in self.block_table or self.request_location.get(rid) == BlockLocation.GPU, \
            f"Request {rid} is on CPU. Migrate to GPU first."
        if num_blocks is None:
            if isinstance(request, str):
                raise ValueError("allocate_blocks: a plain request id needs an explicit num_blocks")
            num_blocks = self.get_num_blocks_needed(request)
        if rid not in self.block_table:
            self.block_table[rid] = self._get_free_blocks(num_blocks, BlockLocation.GPU)
            self.request_location[rid] = BlockLocation.GPU
        else:
            cur = len(self.block_table[rid])
            if cur < num_blocks:
                self.block_table[rid] += self._get_free_blocks(num_blocks - cur, BlockLocation.GPU)
        return self.block_table[rid]

    def allocate_blocks_batched(self, requests: Iterable[Any]) -> None:
        for request in requests:
            self.allocate_blocks(request)

    def expand_blocks_for_seq_len(self, request_id: str, expanded_seq_len: int) -> List[int]:
        """Grow a table to cover a longer sequence (vision tokens spliced in, :216-245)."""
        if request_id not in self.block_table:
            raise ValueError(f"Request {request_id} not allocated")
        needed = self.get_num_blocks_needed(expanded_seq_len)
        cur = len(self.block_table[request_id])
        if cur < needed:
            self.block_table[request_id] += self._get_free_blocks(needed - cur, BlockLocation.GPU)
        return self.block_table[request_id]

    def append_blocks(self, request: Any) -> None:
        rid = _request_id(request)
        assert rid in self.block_table, f"Request {rid} not allocated yet"
        extra = self.get_num_append_blocks_needed(request)
        if extra > 0:
            self.block_table[rid].extend(self._get_free_blocks(extra, BlockLocation.GPU))

    def free_blocks(self, request_id: str) -> None:
        assert request_id in self.block_table, f"Request {request_id} not allocated"
        blocks = self.block_table.pop(request_id)
        if self.request_location.pop(request_id) == BlockLocation.GPU:
            self.free_gpu_blocks_list += blocks
        else:
            self.free_cpu_blocks_list += blocks

    def free_blocks_batched(self, requests: Iterable[RequestLike]) -> None:
        for request in requests:
            rid = _request_id(request)
            if rid in self.block_table:
                self.free_blocks(rid)

    # ----- swapping (block_manager.py:305-377) --------------------------------------------
    def _move_request(self, request_id: str, to_gpu: bool) -> Tuple[List[int], List[int]]:
        here = BlockLocation.CPU if to_gpu else BlockLocation.GPU
        there = BlockLocation.GPU if to_gpu else BlockLocation.CPU
        assert request_id in self.block_table, f"request {request_id} not allocated"
        assert self.request_location[request_id] == here, f"request {request_id} is on {there} now"
        old = self.block_table[request_id]
        new = self._get_free_blocks(len(old), there)
        (self.swapping_cpu_blocks_list if to_gpu else self.swapping_gpu_blocks_list).extend(old)
        self.block_table[request_id] = new
        self.request_location[request_id] = there
        return old, new

    def swap_out(self, request_id: str) -> Tuple[List[int], List[int]]:
        """Bookkeeping only: returns (gpu blocks to read, cpu blocks to write)."""
        return self._move_request(request_id, to_gpu=False)

    def swap_in(self, request_id: str) -> Tuple[List[int], List[int]]:
        """Bookkeeping only: returns (cpu blocks to read, gpu blocks to write)."""
        return self._move_request(request_id, to_gpu=True)

    def swap_requests(self, request_ids: List[str], is_swap_in: bool) -> Tuple[List[int], List[int]]:
        """Move the requests' tables to the other tier and have the workers copy the blocks: one
        ``swap_blocks(request_ids, source_ids, target_ids, is_swap_in)`` call with the concatenated
        tables. Returns the two id lists."""
        source_block_ids: List[int] = []
        target_block_ids: List[int] = []
        for request_id in request_ids:
            old, new = self._move_request(request_id, to_gpu=is_swap_in)
            source_block_ids += old
            target_block_ids += new
        self._call_workers("swap_blocks", request_ids, source_block_ids, target_block_ids, is_swap_in)
        self.swap_count += 1
        return source_block_ids, target_block_ids

    def swap_in_requests(self, request_ids: List[str]) -> Tuple[List[int], List[int]]:
        return self.swap_requests(request_ids, is_swap_in=True)

    def swap_out_requests(self, request_ids: List[str]) -> Tuple[List[int], List[int]]:
        return self.swap_requests(request_ids, is_swap_in=False)

    def clear_request_resource(self, request_id: str) -> None:
        """A finished or aborted request: the workers drop its swap event (:394-403)."""
        self._call_workers("clear_request_resource", request_id)

    def clear_request_resource_batched(self, request_ids: Iterable[str]) -> None:
        for request_id in request_ids:
            self.clear_request_resource(request_id)

    def wait_for_all_swap_in(self) -> None:
        self._call_workers("wait_for_all_swap_in")

    def wait_for_all_swap_out(self) -> None:
        self._call_workers("wait_for_all_swap_out")

    # ----- statistics (block_manager.py:417-441) ---------------------------------------------
    def get_block_usage(self) -> Dict[str, str]:
        cpu_used = self.max_num_cpu_blocks - self.get_num_avail_cpu_blocks()
        gpu_used = self.max_num_gpu_blocks - self.get_num_avail_gpu_blocks()

        def share(n: int, d: int) -> str:
            return f"{round(n / d * 100) if d else 0}% ({n}/{d})"

        return {"gpu": share(gpu_used, self.max_num_gpu_blocks), "cpu": share(cpu_used, self.max_num_cpu_blocks),
                "swap": f"{len(self.swapping_gpu_blocks_list)} -> {len(self.swapping_cpu_blocks_list)}",
                "#req": f"{len(self.block_table)}"}

    def print_block_usage(self) -> None:
        usage = self.get_block_usage()
        print(f"({self.stage}) Block usage: GPU={usage['gpu']}, CPU={usage['cpu']}, "
              f"Swapping={usage['swap']}, Requests={usage['#req']}")

    # ----- pool tensors sized for a batch (block_manager.py:443-485) ---------------------------
    def create_kv_cache_tensors(self, batched_requests: Any, num_layers: int, num_heads: int, head_size: int,
                                dtype: Any, device: str = "cuda") -> List[Any]:
        """One ``[2, max_blocks, block_size, num_heads, head_size]`` tensor per layer, ``max_blocks`` = the most
        blocks any request of the batch needs: the layout every kernel of this package takes as a pool.
        ``batched_requests`` is a BatchedRequests-like object (``.requests``) or an iterable of requests."""
        import torch

        max_blocks_needed = self.get_max_blocks_needed(batched_requests)
        shape = (2, max_blocks_needed, self.block_size, num_heads, head_size)
        return [torch.empty(shape, dtype=dtype, device=device) for _ in range(num_layers)]


class VisionBlockManager(BlockManager):
    """Block tables of the vision-embedding pool (block_manager.py:504-543): a fixed number of
    embedding tokens per image, rounded up to blocks per image."""

    def __init__(self, *args, embedding_tokens_per_image: int = 576, **kwargs):
        super().__init__(*args, **kwargs)
        self.embedding_tokens_per_image = embedding_tokens_per_image

    def get_num_blocks_needed(self, request: Union[int, Any]) -> int:
        if isinstance(request, int):
            return super().get_num_blocks_needed(request)
        images = getattr(request, "images", None)
        if not images:
            return 0
        per_image = (self.embedding_tokens_per_image + self.block_size - 1) // self.block_size
        return len(images) * per_image
