"""KVWorker — the KV data-path surface of the reference's V0Worker on one MI355X.

Method names, argument order, return shapes and error behaviour follow
``elasticmm/engine/v0/worker.py`` (the class ``V0Worker``), restricted to the
methods that touch KV / vision-embedding tensors:

  extract_kv_blocks / write_kv_blocks / get_kv_cache_layout   worker.py:578-647
  p2p_send_kv / p2p_recv_kv                                   worker.py:665-731
  p2p_coordinated_transfer_kv                                 worker.py:733-871
  p2p_pull_kv / p2p_serve_kv                                  worker.py:873-937
  collective_transfer_kv                                      worker.py:939-1005
  extract_vision_blocks / write_vision_blocks                 worker.py:1007-1036
  init_kvcache (pool allocation only)                         worker.py:358-418
  swap_blocks / wait_for_all_swap_in / wait_for_all_swap_out  worker.py:467-526

Model loading, Ray actor plumbing and step_* execution are not part of this
class. The cross-GPU hop (``torch.distributed.send/recv``) is replaced by a
``LoopbackLink``: a same-device FIFO that hands the sender's transfer buffer to
the receiver, which unpacks it into its own, independently allocated pool.
Where the reference loops over layers with one gather / scatter launch each,
this class issues one kernel launch for all layers.
"""
from __future__ import annotations

import collections
import math
import time
from typing import Any, Deque, Dict, List, Optional, Sequence, Tuple

import torch

from . import kv_ops
from .kv_ops import PoolView

_DTYPES = {
    "float16": torch.float16, "half": torch.float16, "fp16": torch.float16,
    "bfloat16": torch.bfloat16, "bf16": torch.bfloat16,
    "float32": torch.float32, "fp32": torch.float32,
}


class LoopbackLink:
    """Same-device stand-in for the global NCCL group: per (src, dst, tag) FIFOs of
    device tensors. ``send`` enqueues a tensor, ``recv`` dequeues it; both sides run
    on the same HIP stream order, so no extra synchronisation is needed.

    Every message may carry the id of the transfer it belongs to (one id for the L
    per-layer messages of one send). A receiver that gives up in the middle of a
    transfer (deadline, shape mismatch) discards the transfer's remaining messages by
    that id, so that the next transfer between the same ranks does not start with
    stale layers."""

    def __init__(self, world_size: int = 2):
        self.world_size = world_size
        self._queues: Dict[Tuple[int, int, int], Deque[Tuple[Optional[int], torch.Tensor]]] = \
            collections.defaultdict(collections.deque)
        self._next_transfer_id = 0

    def new_transfer_id(self) -> int:
        self._next_transfer_id += 1
        return self._next_transfer_id

    def send(self, tensor: torch.Tensor, src: int, dst: int, tag: int = 0, transfer_id: Optional[int] = None) -> None:
        if not (0 <= dst < self.world_size):
            raise ValueError(f"Invalid dst rank: {dst} (world_size={self.world_size})")
        self._queues[(src, dst, tag)].append((transfer_id, tensor))

    def recv_with_id(self, src: int, dst: int, tag: int = 0) -> Tuple[Optional[int], torch.Tensor]:
        q = self._queues[(src, dst, tag)]
        if not q:
            raise RuntimeError(f"no message pending from rank {src} to rank {dst} (tag {tag})")
        return q.popleft()

    def recv(self, src: int, dst: int, tag: int = 0) -> torch.Tensor:
        return self.recv_with_id(src, dst, tag)[1]

    def head_id(self, src: int, dst: int, tag: int = 0) -> Optional[int]:
        """Transfer id of the next message of this FIFO (None if it is empty or the message has none)."""
        q = self._queues[(src, dst, tag)]
        return q[0][0] if q else None

    def pending(self, src: int, dst: int, tag: int = 0) -> int:
        return len(self._queues[(src, dst, tag)])

    def discard(self, src: int, dst: int, transfer_id: Optional[int]) -> int:
        """Drop every queued message of transfer ``transfer_id`` from ``src`` to ``dst`` (all tags).
        Returns the number of messages dropped."""
        if transfer_id is None:
            return 0
        dropped = 0
        for (s, d, _), q in self._queues.items():
            if s == src and d == dst and q:
                kept = [m for m in q if m[0] != transfer_id]
                dropped += len(q) - len(kept)
                q.clear()
                q.extend(kept)
        return dropped

    def drop_pending(self, src: int, dst: int) -> int:
        """Drop everything queued from ``src`` to ``dst`` (all tags, all transfers)."""
        dropped = 0
        for (s, d, _), q in self._queues.items():
            if s == src and d == dst:
                dropped += len(q)
                q.clear()
        return dropped


def _hip_runtime():
    """The HIP runtime torch itself uses (torch ships its own copy next to its libraries)."""
    import ctypes
    import os

    bundled = os.path.join(os.path.dirname(torch.__file__), "lib", "libamdhip64.so")
    rt = ctypes.CDLL(bundled if os.path.exists(bundled) else "libamdhip64.so")
    rt.hipMalloc.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_size_t]
    rt.hipMalloc.restype = ctypes.c_int
    rt.hipFree.argtypes = [ctypes.c_void_p]
    rt.hipFree.restype = ctypes.c_int
    rt.hipGetLastError.restype = ctypes.c_int
    return rt, ctypes


def allocate_layers_spread(num_layers: int, layer_shape: Sequence[int], dtype: torch.dtype, device: torch.device,
                           stripes: int = 4, reserve_bytes: int = 8 << 30) -> List[torch.Tensor]:
    """Allocate the L layer tensors of a pool in ``stripes`` allocations that lie far apart in device memory;
    layer l goes to stripe ``l % stripes``, so consecutive layers are far apart as well.

    Why: on MI355X the scattered 16 KiB writes of unpack / copy_blocks run at 5.4 TB/s when a launch's
    destinations all lie in one large region of device memory and at 6.3 TB/s when they reach more than one
    (the regions are tens of GiB long; a pool of about 50 GiB allocated in one piece often lies inside a single
    one). A pool that fills most of the device spans them anyway; for a smaller pool the stripes are pushed
    apart by allocating a temporary spacer after each stripe (the free memory divided by the number of stripes)
    and releasing the spacers at the end. Nothing is shared with other pools: every pool is allocated by its
    own call. With too little free memory for spacers the stripes are simply allocated one after the other."""
    device = torch.device(device)
    stripes = max(1, min(int(stripes), num_layers))
    layer_elems = 1
    for d in layer_shape:
        layer_elems *= int(d)
    elem = torch.empty((), dtype=dtype).element_size()
    need = num_layers * layer_elems * elem
    counts = [len(range(s, num_layers, stripes)) for s in range(stripes)]
    with torch.cuda.device(device):
        free, _ = torch.cuda.mem_get_info()
        gap = max(0, (free - need - reserve_bytes) // stripes)
        gap -= gap % (2 << 20)
        rt, ctypes = _hip_runtime()
        spacers, parts = [], []
        try:
            for s in range(stripes):
                parts.append(torch.empty(counts[s] * layer_elems, dtype=dtype, device=device))
                if gap > 0 and s + 1 < stripes:
                    ptr = ctypes.c_void_p()
                    if rt.hipMalloc(ctypes.byref(ptr), gap) != 0:
                        rt.hipGetLastError()  # clear it: the next launch check must not see this failure
                        break  # no room for this spacer: the remaining stripes follow directly
                    spacers.append(ptr)
        finally:
            for ptr in spacers:
                rt.hipFree(ptr)
    while len(parts) < stripes:
        parts.append(torch.empty(counts[len(parts)] * layer_elems, dtype=dtype, device=device))
    return [parts[l % stripes][(l // stripes) * layer_elems:(l // stripes + 1) * layer_elems].view(tuple(layer_shape))
            for l in range(num_layers)]


class KVWorker:
    """Owns one block pool on one GPU and moves blocks in and out of it."""

    def __init__(self, worker_id: int = 0, device: str = "cuda:0", block_size: int = 16,
                 link: Optional[LoopbackLink] = None, global_rank: Optional[int] = None):
        self.worker_id = worker_id
        self.device = torch.device(device)
        self.block_size = block_size
        self.kv_cache: Optional[List[torch.Tensor]] = None
        self.ve_cache: Optional[Dict[str, torch.Tensor]] = None
        self._ve_sources: Dict[str, Any] = {}
        self._pool: Optional[PoolView] = None
        self.link = link
        self.global_rank = global_rank
        self.nccl_pg_initialized = link is not None and global_rank is not None
        self.peers: Dict[int, "KVWorker"] = {}
        # CPU swap tier (worker.py:98-108): created lazily, they need a GPU
        self.kv_swap: Optional[List[torch.Tensor]] = None
        self._swap_pool: Optional[PoolView] = None
        self.swap_in_stream: Optional[torch.cuda.Stream] = None
        self.swap_out_stream: Optional[torch.cuda.Stream] = None
        self.swap_event_table: Dict[str, torch.cuda.Event] = {}
        self.latest_swap_in_event: Optional[torch.cuda.Event] = None
        self.latest_swap_out_event: Optional[torch.cuda.Event] = None
        # device-resident block tables are trusted (ids out of range are skipped by the kernels); set this to have
        # extract_kv_blocks / write_kv_blocks validate them first and raise IndexError (costs a synchronisation)
        self.strict_device_tables = False
        self.last_sent_transfer_id: Optional[int] = None

    # ----- pool -----------------------------------------------------------
    def init_kvcache(self, num_gpu_blocks: int, num_cpu_blocks: int = 0, *, num_layers: int, num_kv_heads: int,
                     head_size: int, dtype: torch.dtype = torch.bfloat16, monolithic: bool = True,
                     spread_stripes: int = 0) -> List[int]:
        """Allocate the pool: L tensors ``[2, num_gpu_blocks, block_size, num_kv_heads, head_size]``
        (worker.py:388-394). With ``monolithic`` the L tensors are views of one
        allocation, which keeps the list API and lets the whole pool be one HBM
        region; otherwise each layer is its own allocation as vLLM's CacheEngine does.
        ``spread_stripes = k > 1`` places the layers in k allocations spread over the device's
        free memory (see ``allocate_layers_spread``)."""
        shape = (2, num_gpu_blocks, self.block_size, num_kv_heads, head_size)
        if spread_stripes > 1:
            layers = allocate_layers_spread(num_layers, shape, dtype, self.device, spread_stripes)
        elif monolithic:
            whole = torch.empty((num_layers,) + shape, dtype=dtype, device=self.device)
            layers = list(whole.unbind(0))
        else:
            layers = [torch.empty(shape, dtype=dtype, device=self.device) for _ in range(num_layers)]
        self.bind_kv_cache(layers)
        if num_cpu_blocks > 0:
            cpu_shape = (2, num_cpu_blocks, self.block_size, num_kv_heads, head_size)
            self.bind_kv_swap([torch.empty(cpu_shape, dtype=dtype, pin_memory=True) for _ in range(num_layers)])
        return []  # placeholder for an IPC handle, as in the reference (worker.py:418)

    def bind_kv_cache(self, kv_cache: Sequence[torch.Tensor]) -> None:
        """Adopt an existing pool (e.g. the list vLLM's CacheEngine allocated)."""
        self.kv_cache = list(kv_cache)
        self._pool = PoolView(self.kv_cache)

    def bind_kv_swap(self, kv_swap: Sequence[torch.Tensor]) -> None:
        """Adopt a CPU swap pool: L pinned host tensors ``[2, num_cpu_blocks, bs, H, D]`` (the
        layout of vLLM's ``cpu_cache``, worker.py:389)."""
        self.kv_swap = list(kv_swap)
        self._swap_pool = PoolView(self.kv_swap, pinned_host_for=self.device)

    def init_vecache(self, num_gpu_blocks: int = 0, num_cpu_blocks: int = 0) -> List[int]:
        """Vision embeddings are kept per request id (worker.py:431-437)."""
        self.ve_cache = {}
        self._ve_sources = {}
        self.ve_cache_capacity = num_gpu_blocks
        return []

    @property
    def pool(self) -> PoolView:
        if self._pool is None:
            raise RuntimeError("KV cache not initialized")
        return self._pool

    # ----- extract / write (worker.py:578-647) ------------------------------
    def extract_kv_blocks(self, block_indices: List[int]) -> torch.Tensor:
        """-> ``[num_layers, 2, n, block_size, num_heads, head_size]``, one launch."""
        pool = self._pool
        if self.kv_cache is None or pool is None:
            raise RuntimeError("KV cache not initialized")
        return kv_ops.kv_pack(pool, block_indices, strict=self.strict_device_tables)

    def write_kv_blocks(self, block_indices: List[int], kv_data: torch.Tensor) -> None:
        pool = self._pool
        if self.kv_cache is None or pool is None:
            raise RuntimeError("KV cache not initialized")
        assert kv_data.shape[2] == len(block_indices), \
            f"Block count mismatch: {kv_data.shape[2]} vs {len(block_indices)}"
        if kv_data.dtype != pool.dtype:
            kv_data = kv_data.to(pool.dtype)
        if kv_data.device != self.device:
            kv_data = kv_data.to(self.device)
        kv_ops.kv_unpack(pool, block_indices, kv_data, strict=self.strict_device_tables)

    def get_kv_cache_layout(self) -> Dict[str, Any]:
        if not self.kv_cache:
            return {}
        sample_layer = self.kv_cache[0]
        return {
            "num_layers": len(self.kv_cache),
            "block_size": sample_layer.shape[2],
            "num_heads": sample_layer.shape[3],
            "head_size": sample_layer.shape[4],
            "dtype": str(sample_layer.dtype).split(".")[-1],
        }

    # ----- P2P (worker.py:649-937) over the loopback link -------------------
    def init_global_nccl(self) -> bool:
        return bool(self.nccl_pg_initialized)

    def get_global_rank(self) -> int:
        return self.global_rank if self.global_rank is not None else -1

    def _layer_bytes(self, n: int) -> int:
        return self.pool.num_kv * n * self.pool.chunk_bytes

    def p2p_send_kv(self, dst_rank: int, block_indices: List[int]) -> Dict[str, Any]:
        """Pack all layers with one launch, then hand the link one ``[2, n, bs, H, D]``
        message per layer (views of the one transfer buffer), as the reference sends
        one message per layer."""
        if not self.nccl_pg_initialized:
            return {"error": "Global NCCL not initialized", "bytes": 0, "blocks": 0}
        try:
            packed = kv_ops.kv_pack(self.pool, block_indices)
            total_bytes = 0
            transfer_id = self.link.new_transfer_id()
            try:
                for l in range(self.pool.num_layers):
                    layer_data = packed[l]
                    self.link.send(layer_data, src=self.global_rank, dst=dst_rank, transfer_id=transfer_id)
                    total_bytes += layer_data.numel() * layer_data.element_size()
            except Exception:
                self.link.discard(self.global_rank, dst_rank, transfer_id)  # no half-sent transfer stays queued
                raise
            torch.cuda.synchronize(self.device)
            # the dict keeps the reference's shape; the id of the transfer just sent is left here so that a caller
            # can drop exactly this transfer's messages from the link if the receiving side never takes them
            self.last_sent_transfer_id = transfer_id
            return {"bytes": total_bytes, "blocks": len(block_indices)}
        except Exception as e:  # transport failures are reported, not raised (worker.py:686-691)
            error_msg = f"NCCL send failed: {type(e).__name__}: {str(e)}"
            return {"error": error_msg, "bytes": 0, "blocks": 0}

    def _recv_layers(self, src_rank: int, block_indices: List[int], tagged: bool = False,
                     deadline: Optional[Tuple[float, float]] = None) -> Any:
        """Receive L per-layer messages and scatter them. Messages that are the
        consecutive slices of one transfer buffer are scattered with one launch."""
        pool = self.pool
        n = len(block_indices)
        layer_shape = (pool.num_kv, n) + pool.block_shape
        msgs: List[torch.Tensor] = []
        # the transfer this call consumes: on any early exit its remaining per-layer messages are
        # dropped from the link, so that the next receive does not scatter stale layers
        transfer_id = self.link.head_id(src_rank, self.global_rank, 0)
        complete = False
        try:
            for layer_idx in range(pool.num_layers):
                if deadline is not None and time.time() - deadline[0] > deadline[1]:
                    return layer_idx
                tid, m = self.link.recv_with_id(src=src_rank, dst=self.global_rank, tag=layer_idx if tagged else 0)
                if layer_idx == 0:
                    transfer_id = tid
                elif tid != transfer_id:
                    raise RuntimeError(f"layer {layer_idx}: message of transfer {tid} inside transfer {transfer_id}")
                if tuple(m.shape) != layer_shape:
                    raise RuntimeError(f"layer {layer_idx}: received {tuple(m.shape)}, expected {layer_shape}")
                msgs.append(m)
            complete = True
        finally:
            if not complete:
                self.link.discard(src_rank, self.global_rank, transfer_id)
        total_bytes = sum(m.numel() * m.element_size() for m in msgs)
        step = self._layer_bytes(n)
        whole = msgs[0]._base if msgs else None
        fused = (whole is not None and whole.is_contiguous()
                 and whole.numel() == sum(m.numel() for m in msgs)
                 and all(m._base is whole and m.is_contiguous()
                         and m.data_ptr() == whole.data_ptr() + i * step for i, m in enumerate(msgs)))
        if fused:
            kv_ops.kv_unpack(pool, block_indices, whole)
        else:
            idx = kv_ops.block_index_tensor(block_indices, pool.num_blocks, pool.device)
            for l, m in enumerate(msgs):
                kv_ops.kv_unpack(PoolView([pool.layers[l]]), idx, m)
        return {"bytes": total_bytes}

    def p2p_recv_kv(self, src_rank: int, block_indices: List[int]) -> Dict[str, Any]:
        if not self.nccl_pg_initialized:
            return {"error": "Global NCCL not initialized", "bytes": 0, "blocks": 0}
        try:
            res = self._recv_layers(src_rank, block_indices)
            torch.cuda.synchronize(self.device)
            return {"bytes": res["bytes"], "blocks": len(block_indices)}
        except Exception as e:
            error_msg = f"NCCL recv failed: {type(e).__name__}: {str(e)}"
            return {"error": error_msg, "bytes": 0, "blocks": 0}

    def p2p_coordinated_transfer_kv(self, src_worker_ref: Any, src_rank: int, src_blocks: List[int],
                                    dst_blocks: List[int], timeout: float = 10.0) -> Dict[str, Any]:
        """Called on the destination: triggers the source's send, receives and scatters.
        ``src_worker_ref`` is the source ``KVWorker`` (the reference passes a Ray actor
        handle and calls ``.p2p_send_kv.remote``)."""
        if not self.nccl_pg_initialized:
            raise RuntimeError("Destination worker: Global NCCL not initialized")
        if len(src_blocks) != len(dst_blocks):
            raise ValueError(f"Block count mismatch: src={len(src_blocks)}, dst={len(dst_blocks)}")
        if len(src_blocks) == 0:
            return {"bytes": 0, "blocks": 0, "error": "No blocks to transfer"}
        if src_rank < 0 or src_rank >= self.link.world_size:
            raise ValueError(f"Invalid src_rank: {src_rank} (world_size={self.link.world_size})")
        start_time = time.time()
        try:
            send_result = src_worker_ref.p2p_send_kv(self.global_rank, src_blocks)
            if "error" in send_result:
                return {"error": f"Send error: {send_result['error']}", "bytes": 0, "blocks": 0,
                        "elapsed": time.time() - start_time}
            res = self._recv_layers(src_rank, dst_blocks, deadline=(start_time, timeout))
            if isinstance(res, int):
                return {"error": f"Transfer timeout after {timeout}s at layer {res}/{len(self.kv_cache)}",
                        "bytes": 0, "blocks": 0, "elapsed": time.time() - start_time}
            torch.cuda.synchronize(self.device)
            elapsed = time.time() - start_time
            total_bytes = res["bytes"]
            if send_result["bytes"] != total_bytes:
                print(f"[KVWorker] Warning: Transfer size mismatch: expected {total_bytes}, got {send_result['bytes']}")
            return {"bytes": total_bytes, "blocks": len(dst_blocks), "elapsed": elapsed,
                    "method": "coordinated_single_call"}
        except Exception as e:
            elapsed = time.time() - start_time
            error_msg = f"NCCL coordinated transfer failed after {elapsed:.2f}s: {type(e).__name__}: {str(e)}"
            return {"error": error_msg, "bytes": 0, "blocks": 0, "elapsed": elapsed}

    def p2p_pull_kv(self, src_rank: int, src_blocks: List[int], dst_blocks: List[int]) -> Dict[str, Any]:
        """Receiver-initiated transfer: send the request (block ids, tag 999), let the
        source serve it, receive layer messages tagged by layer index."""
        if not self.nccl_pg_initialized:
            raise RuntimeError("Global NCCL not initialized")
        request_tensor = torch.full((1024,), -1, dtype=torch.long)
        if len(src_blocks) > 1024:
            raise ValueError("at most 1024 blocks per pull request")
        request_tensor[:len(src_blocks)] = torch.as_tensor(list(src_blocks), dtype=torch.long)
        self.link.send(request_tensor.to(self.device), src=self.global_rank, dst=src_rank, tag=999)
        server = self.peers.get(src_rank)
        if server is not None:  # the reference's source actor runs p2p_serve_kv concurrently
            server.p2p_serve_kv(self.global_rank)
        res = self._recv_layers(src_rank, dst_blocks, tagged=True)
        torch.cuda.synchronize(self.device)
        return {"bytes": res["bytes"], "blocks": len(dst_blocks)}

    def p2p_serve_kv(self, requester_rank: int) -> Dict[str, Any]:
        """Serve a pull request: a fixed 1024-slot int64 request padded with -1
        (worker.py:920-925). The ids stay on the device; only their count is read back."""
        if not self.nccl_pg_initialized:
            raise RuntimeError("Global NCCL not initialized")
        request_tensor = self.link.recv(src=requester_rank, dst=self.global_rank, tag=999)
        block_idx = request_tensor[request_tensor >= 0]
        n = int(block_idx.numel())
        packed = kv_ops.kv_pack(self.pool, block_idx)
        total_bytes = 0
        transfer_id = self.link.new_transfer_id()
        for layer_idx in range(self.pool.num_layers):
            layer_data = packed[layer_idx]
            self.link.send(layer_data, src=self.global_rank, dst=requester_rank, tag=layer_idx,
                           transfer_id=transfer_id)
            total_bytes += layer_data.numel() * layer_data.element_size()
        torch.cuda.synchronize(self.device)
        return {"bytes": total_bytes, "blocks": n}

    def collective_transfer_kv(self, group_name: str, root: int, block_indices: List[int],
                               tensor_shape: Sequence[int], dtype: str, mode: str) -> Dict[str, Any]:
        """Flat-buffer form (worker.py:939-1005): the sender packs and publishes one flat
        tensor; the receiver takes it, views it as ``tensor_shape`` and scatters it."""
        normalized_dtype = dtype.replace("torch.", "").lower()
        if normalized_dtype not in _DTYPES:
            raise ValueError(f"[KVWorker] Unsupported dtype for collective transfer: {dtype}")
        torch_dtype = _DTYPES[normalized_dtype]
        tensor_shape = tuple(int(dim) for dim in tensor_shape)
        if self.link is None:
            raise RuntimeError("no link attached")
        tag = hash(group_name) & 0x7FFFFFFF
        if mode == "send":
            kv_tensor = self.extract_kv_blocks(block_indices).contiguous()
            flat_tensor = kv_tensor.view(-1).to(dtype=torch_dtype)
            for dst in range(self.link.world_size):
                if dst != root:
                    self.link.send(flat_tensor, src=root, dst=dst, tag=tag)
            bytes_transferred = flat_tensor.numel() * flat_tensor.element_size()
        elif mode == "recv":
            numel = math.prod(tensor_shape)
            flat_tensor = self.link.recv(src=root, dst=self.global_rank, tag=tag)
            if flat_tensor.numel() != numel or flat_tensor.dtype != torch_dtype:
                raise RuntimeError("broadcast payload does not match tensor_shape / dtype")
            kv_tensor = flat_tensor.view(tensor_shape)
            self.write_kv_blocks(block_indices, kv_tensor)
            bytes_transferred = flat_tensor.numel() * flat_tensor.element_size()
        else:
            raise ValueError(f"[KVWorker] Unknown collective transfer mode: {mode}")
        torch.cuda.synchronize(self.device)
        return {"bytes": bytes_transferred, "mode": mode}

    # ----- GPU <-> CPU swap (worker.py:467-526) ------------------------------
    def wait_for_all_swap_out(self) -> None:
        if self.latest_swap_out_event:
            self.latest_swap_out_event.wait()

    def wait_for_all_swap_in(self) -> None:
        if self.latest_swap_in_event:
            self.latest_swap_in_event.wait()

    def swap_blocks(self, request_ids: List[str], source_block_ids: List[int], target_block_ids: List[int],
                    is_swap_in: bool) -> None:
        """Copy blocks between the CPU swap pool and the GPU pool: swap-in moves CPU block
        ``source_block_ids[i]`` to GPU block ``target_block_ids[i]``, swap-out the other way.
        One kernel per call reads / writes the pinned host pool directly over PCIe (all layers,
        K and V), on the swap-in / swap-out side stream. A request's swaps are ordered by its
        event; the event is recorded after the copy so that waiting on it means the data has
        arrived (the reference records it before issuing the copy, worker.py:499-500, and then
        indexes the per-layer list as one tensor, :521/:526, which cannot run)."""
        if self.kv_cache is None or self.kv_swap is None:
            raise RuntimeError("KV cache / swap pool not initialized")
        if len(source_block_ids) != len(target_block_ids):
            raise ValueError(f"Block count mismatch: src={len(source_block_ids)}, dst={len(target_block_ids)}")
        if self.swap_in_stream is None:
            self.swap_in_stream = torch.cuda.Stream(self.device)
            self.swap_out_stream = torch.cuda.Stream(self.device)
        stream = self.swap_in_stream if is_swap_in else self.swap_out_stream
        # the side stream starts after what the caller has queued so far (blocks being swapped
        # out must have been written; blocks being swapped in must no longer be read)
        stream.wait_stream(torch.cuda.current_stream(self.device))
        for request_id in request_ids:
            if request_id in self.swap_event_table:
                self.swap_event_table[request_id].wait(stream)
        with torch.cuda.stream(stream):
            if is_swap_in:
                kv_ops.kv_migrate(self._swap_pool, source_block_ids, self.pool, target_block_ids)
            else:
                kv_ops.kv_migrate(self.pool, source_block_ids, self._swap_pool, target_block_ids)
            event = torch.cuda.Event()
            event.record(stream)
        for request_id in request_ids:
            self.swap_event_table[request_id] = event
        if is_swap_in:
            self.latest_swap_in_event = event
        else:
            self.latest_swap_out_event = event

    def clear_request_resource(self, request_id: str) -> None:
        """worker.py:528-532: forget the request's swap event."""
        self.swap_event_table.pop(request_id, None)

    def clear_request_resource_batched(self, request_ids: List[str]) -> None:
        """worker.py:534-537."""
        for request_id in request_ids:
            self.clear_request_resource(request_id)

    def clear_all_requests(self) -> None:
        """worker.py:1114-1132: drop every cached vision embedding (before a role switch); the KV pool
        stays allocated, its blocks belong to the block manager."""
        if self.ve_cache is not None:
            self.ve_cache.clear()
        self._ve_sources.clear()
        self.swap_event_table.clear()

    # ----- shapes (worker.py:1038-1064) ---------------------------------------
    def get_kv_cache_shape(self) -> tuple:
        """``(num_layers, 2, num_blocks, block_size, num_kv_heads, head_size)``, or ``()`` without a pool.
        The reference asks the per-layer list for ``.shape`` (worker.py:1042), which a list does not have; this
        is the shape its 6-D consumers (nccl_transfer.py:215) expect."""
        if self.kv_cache is None:
            return ()
        return (len(self.kv_cache),) + tuple(self.kv_cache[0].shape)

    def get_ve_cache_shape(self) -> tuple:
        """``()``: vision embeddings are kept per request id, not in one tensor (worker.py:431-437)."""
        return ()

    def get_ve_cache_keys(self) -> List[str]:
        return [] if self.ve_cache is None else list(self.ve_cache.keys())

    def get_ve_shape(self, request_id: str) -> Optional[tuple]:
        if self.ve_cache and request_id in self.ve_cache:
            return tuple(self.ve_cache[request_id].shape)
        return None

    # ----- vision embeddings (worker.py:1007-1036, worker_steps.py:252-267) --
    def extract_vision_blocks(self, request_id: str) -> torch.Tensor:
        if self.ve_cache is None:
            raise RuntimeError("Vision embedding cache not initialized")
        if request_id not in self.ve_cache:
            raise KeyError(f"Request {request_id} not found in vision cache")
        return self.ve_cache[request_id]

    def write_vision_blocks(self, request_id: str, ve_data: torch.Tensor) -> None:
        if self.ve_cache is None:
            raise RuntimeError("Vision embedding cache not initialized")
        self.ve_cache[request_id] = ve_data
        self._ve_sources.pop(request_id, None)

    def gather_vision_embeddings(self, request_ids: Sequence[str]) -> Optional[torch.Tensor]:
        """The prefill input built at worker_steps.py:252-267: embeddings of the batch's
        requests that are cached, concatenated on dim 0 (a single tensor passes through).

        ``ve_cache`` stays the plain dict of the reference (callers may assign into it); next to it
        a prepared segment per entry is kept and revalidated by identity, so that the host cost of
        a gather is a few dictionary lookups per request."""
        if self.ve_cache is None:
            return None
        cache, prepared = self.ve_cache, self._ve_sources
        hits = [(r, cache[r]) for r in request_ids if r in cache]
        if not hits:
            return None
        if len(hits) == 1:
            return hits[0][1]
        sources = []
        for r, t in hits:
            s = prepared.get(r)
            if s is None or s.tensor is not t:
                s = kv_ops.RowSource(t)
                if s.tensor is not t:  # a non-contiguous entry: cache its contiguous copy
                    cache[r] = s.tensor
                prepared[r] = s
            sources.append(s)
        if len(prepared) > 2 * len(cache) + 64:  # entries of requests that left the cache
            for r in [r for r in prepared if r not in cache]:
                del prepared[r]
        return kv_ops.concat_row_sources(sources)
