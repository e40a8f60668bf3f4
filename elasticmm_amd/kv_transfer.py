"""KVTransferManager — the caller of the KV data path, same call shape as the reference's
``V0KVTransferManager`` (elasticmm/engine/v0/kv_transfer.py).

What is kept: the method enum (:14-19), the rank-keyed worker registry (:100-168), the
coroutine ``transfer_kv_cache(request_id, src_rank, dst_rank, src_blocks, dst_blocks) -> bool``
that dispatches on the method (:224-262), the statistics that leave out the first (cold-start)
transfer (:82-86, :506-515, :843-859), the metrics callback, and the optional batching that
concatenates several requests' block lists into one transfer (:341-418).

What is different: workers are ``KVWorker`` objects in this process, not Ray actors, so the calls
are plain method calls. The reference's batching path is disabled in the product and its enqueue
code refers to undefined names (:439); here the queue is keyed by (src_rank, dst_rank) and a flush
moves the merged tables with one pack launch and one unpack launch.

The coroutines (``transfer_kv_cache``, ``transfer_vision_embeddings``, ``migrate_requests``) run
their ``*_sync`` bodies on the calling (event-loop) thread without an await point in between. Two
guarantees follow, and callers may rely on both:

* the host bookkeeping of a transfer — block-manager allocations and frees, the batch queue, the
  link's FIFOs and transfer ids — is atomic with respect to every other coroutine of the loop (a
  scheduler coroutine allocating from the same block manager can never be handed the same ids);
* the kernels are launched on the CALLER's current torch stream (torch's current stream is
  per thread), so a transfer is stream-ordered with what the caller queued before and queues
  after it on that stream: when ``migrate_requests`` returns and frees the source blocks, work the
  caller then queues on the same stream cannot overtake the pack that read them. A caller that
  works on other streams orders them itself (``stream.wait_stream``), as with any torch op.

What a transfer costs the loop is launch time (microseconds); the device work itself is
asynchronous except where a worker method synchronises as the reference's does (worker.py:684, :724).
"""
from __future__ import annotations

import time
from enum import Enum
from typing import Any, Callable, Dict, List, Optional, Sequence, Tuple


class TransferMethod(Enum):
    """kv_transfer.py:14-19. CUDA_IPC is the reference's placeholder for a fused device-side
    migration op; here it is the fused same-device ``kv_migrate`` (no transfer buffer)."""
    CUDA_IPC = "cuda_ipc"
    NCCL = "nccl"
    P2P_COPY = "p2p_copy"
    STAGED_COPY = "staged_copy"


class KVTransferManager:
    def __init__(self, transfer_method: TransferMethod = TransferMethod.P2P_COPY, enable_batching: bool = False,
                 batch_size: int = 3, batch_timeout: float = 0.005,
                 metrics_callback: Optional[Callable[..., None]] = None):
        self.transfer_method = transfer_method
        self.enable_batching = enable_batching
        self.metrics_callback = metrics_callback
        self.worker_registry: Dict[int, Any] = {}
        self.rank_to_stage: Dict[int, str] = {}
        self._transfer_queue: Dict[Tuple[int, int], List[Tuple[str, List[int], List[int]]]] = {}
        self._batch_flush_threshold = batch_size
        self._batch_flush_timeout = batch_timeout
        self._last_flush_time: Dict[Tuple[int, int], float] = {}
        # statistics exclude the first transfer (cold start), as in the reference
        self.transfer_count = 0
        self.total_transfer_time = 0.0
        self.total_bytes_transferred = 0
        self.first_transfer_done = False

    def close(self) -> None:
        """Nothing to release (kept for callers that close their managers)."""

    # ----- registry (kv_transfer.py:113-168) ---------------------------------
    def register_workers(self, stage: str, workers: Sequence[Any], global_ranks: Sequence[int]) -> None:
        for worker, rank in zip(workers, global_ranks):
            if worker is not None and rank >= 0:
                self.register_worker(rank, worker, stage)

    def register_worker(self, global_rank: int, worker: Any, stage: str) -> None:
        self.worker_registry[global_rank] = worker
        self.rank_to_stage[global_rank] = stage.lower()

    def unregister_worker(self, global_rank: int) -> None:
        self.worker_registry.pop(global_rank, None)
        self.rank_to_stage.pop(global_rank, None)

    def update_worker_stage(self, global_rank: int, new_stage: str) -> None:
        if global_rank not in self.worker_registry:
            print(f"[KVTransferManager] Warning: Rank {global_rank} not registered")
            return
        self.rank_to_stage[global_rank] = new_stage.lower()

    # ----- transfer (kv_transfer.py:224-262) ----------------------------------
    async def transfer_kv_cache(self, request_id: str, src_rank: int, dst_rank: int, src_blocks: List[int],
                                dst_blocks: List[int]) -> bool:
        return self.transfer_kv_cache_sync(request_id, src_rank, dst_rank, src_blocks, dst_blocks)

    # ----- vision embeddings (kv_transfer.py:264-301, 've' branch of :724-728) ----
    async def transfer_vision_embeddings(self, request_id: str, src_rank: int, src_blocks: List[int],
                                         dst_rank: int, dst_blocks: List[int]) -> bool:
        return self.transfer_vision_embeddings_sync(request_id, src_rank, src_blocks, dst_rank, dst_blocks)

    def transfer_vision_embeddings_sync(self, request_id: str, src_rank: int, src_blocks: List[int],
                                        dst_rank: int, dst_blocks: List[int]) -> bool:
        """Move a request's vision embeddings from the source worker's cache to the destination's.

        The reference routes every method but CUDA_IPC (a placeholder there) to the 've' branch of
        ``_transfer_via_p2p_copy``: ``extract_vision_blocks(request_id)`` on the source,
        ``write_vision_blocks(request_id, data)`` on the destination; the block lists are carried for
        logging only. Its signature still names (stage, worker_id) pairs although its body hands them
        on as ranks (and two arguments too many); here the arguments are the ranks the registry is
        keyed by."""
        src_worker, dst_worker = self._workers(src_rank, dst_rank)
        if src_worker is None:
            return False
        try:
            start_time = time.perf_counter()
            ve_data = src_worker.extract_vision_blocks(request_id)
            dst_worker.write_vision_blocks(request_id, ve_data)
            _ = time.perf_counter() - start_time
            self.transfer_count += 1  # counted, but not reported to the metrics callback (kv only, :743)
            return True
        except Exception as e:
            print(f"[KVTransferManager] P2P copy failed: {e}")
            return False

    def transfer_kv_cache_sync(self, request_id: str, src_rank: int, dst_rank: int, src_blocks: List[int],
                               dst_blocks: List[int]) -> bool:
        if self.transfer_method == TransferMethod.NCCL:
            if self.enable_batching:
                return self._enqueue(request_id, src_rank, dst_rank, src_blocks, dst_blocks)
            return self._transfer_via_p2p(request_id, src_rank, src_blocks, dst_rank, dst_blocks)
        if self.transfer_method == TransferMethod.P2P_COPY:
            return self._transfer_via_p2p_copy(request_id, src_rank, src_blocks, dst_rank, dst_blocks)
        if self.transfer_method == TransferMethod.CUDA_IPC:
            return self._transfer_via_device_migrate(request_id, src_rank, src_blocks, dst_rank, dst_blocks)
        if self.transfer_method == TransferMethod.STAGED_COPY:
            return self._transfer_via_staged_copy(request_id, src_rank, src_blocks, dst_rank, dst_blocks)
        return False

    def _workers(self, src_rank: int, dst_rank: int):
        src_worker = self.worker_registry.get(src_rank)
        dst_worker = self.worker_registry.get(dst_rank)
        if src_worker is None or dst_worker is None:
            print(f"[KVTransferManager] Workers not found: src_rank={src_rank}, dst_rank={dst_rank}")
            return None, None
        return src_worker, dst_worker

    def _account(self, elapsed: float, nbytes: int, num_blocks: int, transfers: int = 1) -> None:
        if not self.first_transfer_done:
            self.first_transfer_done = True
        else:
            self.transfer_count += transfers
            self.total_transfer_time += elapsed
            self.total_bytes_transferred += nbytes
        if self.metrics_callback:
            self.metrics_callback(transfer_time_sec=elapsed, num_blocks=num_blocks)

    def _transfer_via_p2p(self, request_id, src_rank, src_blocks, dst_rank, dst_blocks) -> bool:
        """kv_transfer.py:420-524: one coordinated call on the destination worker."""
        src_worker, dst_worker = self._workers(src_rank, dst_rank)
        if src_worker is None:
            return False
        try:
            start_time = time.perf_counter()
            recv_result = dst_worker.p2p_coordinated_transfer_kv(src_worker, src_rank, src_blocks, dst_blocks,
                                                                 timeout=10.0)
            elapsed = time.perf_counter() - start_time
            if "error" in recv_result:
                print(f"[KVTransferManager] transfer failed for {request_id}: {recv_result.get('error')}")
                return False
            nbytes = recv_result.get("bytes", 0)
            if nbytes == 0:
                return False
            self._account(elapsed, nbytes, len(src_blocks))
            return True
        except Exception as e:  # pre-flight errors of the worker are reported as a failed transfer
            print(f"[KVTransferManager] P2P transfer failed: {e}")
            return False

    def _transfer_via_p2p_copy(self, request_id, src_rank, src_blocks, dst_rank, dst_blocks) -> bool:
        """kv_transfer.py:693-750: extract on the source, write on the destination."""
        src_worker, dst_worker = self._workers(src_rank, dst_rank)
        if src_worker is None:
            return False
        try:
            start_time = time.perf_counter()
            kv_data = src_worker.extract_kv_blocks(src_blocks)
            dst_worker.write_kv_blocks(dst_blocks, kv_data)
            elapsed = time.perf_counter() - start_time
            self.transfer_count += 1
            if self.metrics_callback:
                self.metrics_callback(transfer_time_sec=elapsed, num_blocks=len(src_blocks))
            return True
        except Exception as e:
            print(f"[KVTransferManager] P2P copy failed: {e}")
            return False

    def _transfer_via_device_migrate(self, request_id, src_rank, src_blocks, dst_rank, dst_blocks) -> bool:
        """The slot the reference reserves for a fused device-side op (kv_transfer.py:303-331,
        ``block_migration_ops.migrate_blocks``): pool-to-pool in one launch, both pools on one device."""
        from . import kv_ops

        src_worker, dst_worker = self._workers(src_rank, dst_rank)
        if src_worker is None:
            return False
        try:
            start_time = time.perf_counter()
            kv_ops.kv_migrate(src_worker.pool, src_blocks, dst_worker.pool, dst_blocks)
            elapsed = time.perf_counter() - start_time
            self.transfer_count += 1
            if self.metrics_callback:
                self.metrics_callback(transfer_time_sec=elapsed, num_blocks=len(src_blocks))
            return True
        except Exception as e:
            print(f"[KVTransferManager] device migrate failed: {e}")
            return False

    def _transfer_via_staged_copy(self, request_id, src_rank, src_blocks, dst_rank, dst_blocks) -> bool:
        """Through host memory (kv_transfer.py:821-840, a placeholder that sleeps there): pack on the source, one
        copy into page-locked host memory, one copy onto the destination's device, unpack. For workers whose
        devices cannot reach each other; PCIe-bound."""
        import torch

        src_worker, dst_worker = self._workers(src_rank, dst_rank)
        if src_worker is None:
            return False
        try:
            start_time = time.perf_counter()
            kv_data = src_worker.extract_kv_blocks(src_blocks)
            staged = torch.empty(kv_data.shape, dtype=kv_data.dtype, pin_memory=True)
            staged.copy_(kv_data, non_blocking=True)
            torch.cuda.current_stream(kv_data.device).synchronize()  # the host copy is complete
            dst_worker.write_kv_blocks(dst_blocks, staged.to(dst_worker.device, non_blocking=True))
            elapsed = time.perf_counter() - start_time
            self.transfer_count += 1
            if self.metrics_callback:
                self.metrics_callback(transfer_time_sec=elapsed, num_blocks=len(src_blocks))
            return True
        except Exception as e:
            print(f"[KVTransferManager] staged copy failed: {e}")
            return False

    # ----- migration of whole requests (backend.py:674-737) -----------------------
    async def migrate_requests(self, request_ids: Sequence[str], src_rank: int, src_block_manager: Any,
                               dst_rank: int, dst_block_manager: Any) -> bool:
        return self.migrate_requests_sync(request_ids, src_rank, src_block_manager, dst_rank, dst_block_manager)

    def migrate_requests_sync(self, request_ids: Sequence[str], src_rank: int, src_block_manager: Any,
                              dst_rank: int, dst_block_manager: Any) -> bool:
        """The KV part of the reference's ``migrate_instance`` (elasticmm/engine/v0/backend.py:674-737):
        for every request allocate as many destination blocks as it holds on the source, move its
        blocks, and — only once all requests have moved — free the source blocks. A request without
        blocks is skipped. If an allocation or a transfer fails, the destination blocks taken so far
        are freed, the source is left untouched, and False is returned."""
        moved: List[str] = []

        def roll_back() -> None:
            # with batching the moved requests may still sit in the queue: take them out before
            # their destination blocks go back to the free list, or a later flush would scatter
            # into blocks that belong to nobody (or to another request by then)
            self._purge_queued((src_rank, dst_rank), moved)
            for rid in moved:
                dst_block_manager.free_blocks(rid)

        for request_id in request_ids:
            src_blocks = src_block_manager.get_block_table(request_id)
            if not src_blocks:
                print(f"[KVTransferManager] No blocks found for request {request_id}, skipping")
                continue
            try:
                dst_block_manager.allocate_blocks(request_id, len(src_blocks))
            except Exception as e:
                print(f"[KVTransferManager] Failed to allocate {len(src_blocks)} blocks for {request_id}: {e}")
                roll_back()
                return False
            dst_blocks = dst_block_manager.get_block_table(request_id)
            if not self.transfer_kv_cache_sync(request_id, src_rank, dst_rank, src_blocks, dst_blocks):
                print(f"[KVTransferManager] KV transfer failed for {request_id}")
                dst_block_manager.free_blocks(request_id)
                roll_back()
                return False
            moved.append(request_id)
        if self.enable_batching and not self.flush_transfer_batch(src_rank, dst_rank):
            roll_back()
            return False
        for request_id in moved:
            src_block_manager.free_blocks(request_id)
        return True

    # ----- batching (kv_transfer.py:341-418, :434-462) -------------------------
    def _enqueue(self, request_id, src_rank, dst_rank, src_blocks, dst_blocks) -> bool:
        key = (src_rank, dst_rank)
        if key not in self._transfer_queue:
            self._transfer_queue[key] = []
            self._last_flush_time[key] = time.perf_counter()
        self._transfer_queue[key].append((request_id, list(src_blocks), list(dst_blocks)))
        now = time.perf_counter()
        if (len(self._transfer_queue[key]) >= self._batch_flush_threshold
                or now - self._last_flush_time[key] >= self._batch_flush_timeout):
            self._last_flush_time[key] = now
            return self.flush_transfer_batch(src_rank, dst_rank)
        return True  # queued, flushed later

    def _purge_queued(self, key: Tuple[int, int], request_ids: Sequence[str]) -> int:
        """Remove the queued (not yet flushed) transfers of `request_ids` from the batch queue."""
        queue = self._transfer_queue.get(key)
        if not queue or not request_ids:
            return 0
        gone = set(request_ids)
        kept = [t for t in queue if t[0] not in gone]
        removed = len(queue) - len(kept)
        self._transfer_queue[key] = kept
        return removed

    def flush_transfer_batch(self, src_rank: int, dst_rank: int) -> bool:
        """Merge the queued requests' tables and move them with one send / one receive."""
        key = (src_rank, dst_rank)
        transfers = self._transfer_queue.get(key) or []
        if not transfers:
            return True
        self._transfer_queue[key] = []
        all_src_blocks: List[int] = []
        all_dst_blocks: List[int] = []
        for _, src_blocks, dst_blocks in transfers:
            all_src_blocks.extend(src_blocks)
            all_dst_blocks.extend(dst_blocks)
        src_worker, dst_worker = self._workers(src_rank, dst_rank)
        if src_worker is None:
            return False
        try:
            start_time = time.perf_counter()
            send_result = src_worker.p2p_send_kv(dst_rank, all_src_blocks)
            if "error" in send_result:
                return False
            recv_result = dst_worker.p2p_recv_kv(src_rank, all_dst_blocks)
            if "error" in recv_result:
                # the send went through: what is left of THIS transfer must not stay on the link for the next one
                # (a receive that started has already dropped its remaining layers; one that never started has
                # not). Other transfers between the two ranks, and pull requests, are not touched.
                link = getattr(src_worker, "link", None)
                sent = getattr(src_worker, "last_sent_transfer_id", None)
                if link is not None and sent is not None:
                    link.discard(src_rank, dst_rank, sent)
                return False
            elapsed = time.perf_counter() - start_time
            nbytes = recv_result.get("bytes", 0)
            if nbytes == 0:
                return False
            self.transfer_count += len(transfers)
            self.total_transfer_time += elapsed
            self.total_bytes_transferred += nbytes
            return True
        except Exception as e:
            print(f"[KVTransferManager] Batched transfer failed: {e}")
            return False

    def flush_all(self) -> bool:
        ok = True
        for src_rank, dst_rank in list(self._transfer_queue):
            ok = self.flush_transfer_batch(src_rank, dst_rank) and ok
        return ok

    # ----- statistics (kv_transfer.py:843-859) ---------------------------------
    def get_stats(self) -> Dict[str, Any]:
        return {
            "transfer_count": self.transfer_count,
            "total_transfer_time": self.total_transfer_time,
            "total_bytes_transferred": self.total_bytes_transferred,
            "avg_transfer_time": (self.total_transfer_time / self.transfer_count if self.transfer_count > 0 else 0.0),
        }

    def reset_stats(self) -> None:
        self.transfer_count = 0
        self.total_transfer_time = 0.0
        self.total_bytes_transferred = 0


class KVMigrationManager:
    """Cross-stage moves addressed by (stage, worker id) (kv_transfer.py:867-980, ``V0KVMigrationManager``):
    extract on the source worker, write on the destination worker, for KV blocks and for a request's vision
    embeddings. The reference's worker lookup is a placeholder that finds nobody (:961-969), so its moves always
    report failure; here workers are registered under (stage, worker id). The coroutines run on the calling thread,
    on the caller's current stream, like ``KVTransferManager``'s."""

    def __init__(self):
        self.migration_count = 0
        self.total_migration_time = 0.0
        self._workers_by_stage: Dict[Tuple[str, int], Any] = {}

    def close(self) -> None:
        """Nothing to release."""

    def register_worker(self, stage: str, worker_id: int, worker: Any) -> None:
        self._workers_by_stage[(stage.lower(), worker_id)] = worker

    def unregister_worker(self, stage: str, worker_id: int) -> None:
        self._workers_by_stage.pop((stage.lower(), worker_id), None)

    def _get_worker_ref(self, stage: str, worker_id: int):
        return self._workers_by_stage.get((stage.lower(), worker_id))

    def _pair(self, src_stage, src_worker_id, dst_stage, dst_worker_id):
        src_worker = self._get_worker_ref(src_stage, src_worker_id)
        dst_worker = self._get_worker_ref(dst_stage, dst_worker_id)
        if src_worker is None or dst_worker is None:
            print(f"[KVMigrationManager] Worker not found: src={src_stage}/{src_worker_id}, "
                  f"dst={dst_stage}/{dst_worker_id}")
            return None, None
        return src_worker, dst_worker

    def migrate_kv_blocks_sync(self, request_id: str, src_stage: str, src_worker_id: int, src_blocks: List[int],
                               dst_stage: str, dst_worker_id: int, dst_blocks: List[int]) -> bool:
        start_time = time.time()
        try:
            src_worker, dst_worker = self._pair(src_stage, src_worker_id, dst_stage, dst_worker_id)
            if src_worker is None:
                return False
            kv_data = src_worker.extract_kv_blocks(src_blocks)
            dst_worker.write_kv_blocks(dst_blocks, kv_data)
            self.migration_count += 1
            self.total_migration_time += time.time() - start_time
            return True
        except Exception as e:
            print(f"[KVMigrationManager] KV migration failed: {e}")
            return False

    def migrate_vision_embeddings_sync(self, request_id: str, src_stage: str, src_worker_id: int, dst_stage: str,
                                       dst_worker_id: int) -> bool:
        start_time = time.time()
        try:
            src_worker, dst_worker = self._pair(src_stage, src_worker_id, dst_stage, dst_worker_id)
            if src_worker is None:
                return False
            ve_data = src_worker.extract_vision_blocks(request_id)
            dst_worker.write_vision_blocks(request_id, ve_data)
            self.migration_count += 1
            self.total_migration_time += time.time() - start_time
            return True
        except Exception as e:
            print(f"[KVMigrationManager] Vision embedding migration failed: {e}")
            return False

    async def migrate_kv_blocks(self, request_id: str, src_stage: str, src_worker_id: int, src_blocks: List[int],
                                dst_stage: str, dst_worker_id: int, dst_blocks: List[int]) -> bool:
        return self.migrate_kv_blocks_sync(request_id, src_stage, src_worker_id, src_blocks, dst_stage,
                                           dst_worker_id, dst_blocks)

    async def migrate_vision_embeddings(self, request_id: str, src_stage: str, src_worker_id: int, dst_stage: str,
                                        dst_worker_id: int) -> bool:
        return self.migrate_vision_embeddings_sync(request_id, src_stage, src_worker_id, dst_stage, dst_worker_id)

    def get_stats(self) -> Dict[str, Any]:
        return {
            "migration_count": self.migration_count,
            "total_migration_time": self.total_migration_time,
            "avg_migration_time": (self.total_migration_time / self.migration_count
                                   if self.migration_count > 0 else 0.0),
        }
