"""Tensor-level operators over libemm_kv.so.

Every function launches on torch's current HIP stream of the tensors' device and
returns without synchronising. torch is used for device memory and streams
only; all data movement is done by the HIP kernels of the library.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Union

import numpy as np
import torch

from . import _lib
from ._lib import (EMM_DTYPE_BF16, EMM_DTYPE_F16, EMM_FP8_SATURATE, EMM_MAX_INLINE_IDS, EMM_MAX_LAYERS,
                   EMM_MAX_SEGMENTS, check,
                   ptr_table)

IndexLike = Union[Sequence[int], np.ndarray, torch.Tensor]


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device: torch.device) -> int:
    """hipStream_t of torch's current stream on `device`, as an integer."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


def _require_gpu(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{what}: tensor is on {t.device}; the KV kernels run on the GPU only")


def host_block_ids(block_indices: IndexLike, num_blocks: int) -> Optional[np.ndarray]:
    """Block ids held on the host (Python list, numpy array, CPU tensor) as a contiguous int64 array,
    checked with the semantics torch gives ``tensor[:, idx]`` (worker.py:597, :604): ids in
    [-num_blocks, num_blocks), negatives counted from the end, anything else IndexError.
    None for a device tensor."""
    if isinstance(block_indices, torch.Tensor):
        t = block_indices
        if t.dtype != torch.long:
            raise TypeError(f"block index tensor must be int64, got {t.dtype}")
        if t.is_cuda:
            return None
        arr = t.numpy()
    else:
        arr = np.asarray(block_indices, dtype=np.int64)
    flat_list = arr.ndim == 1 and isinstance(block_indices, (list, tuple))
    arr = np.ascontiguousarray(arr.reshape(-1))
    if arr.size:
        if arr.size <= 64 and flat_list:  # numpy's reductions cost more than the list's
            lo, hi = min(block_indices), max(block_indices)
        else:
            lo, hi = int(arr.min()), int(arr.max())
        if lo < -num_blocks or hi >= num_blocks:
            bad = lo if lo < -num_blocks else hi
            raise IndexError(f"index {bad} is out of bounds for dimension 1 with size {num_blocks}")
        if lo < 0:
            arr = np.where(arr < 0, arr + num_blocks, arr)
    return arr


def block_index_tensor(block_indices: IndexLike, num_blocks: int, device: torch.device) -> torch.Tensor:
    """int64 device tensor of block ids.

    Host ids are checked (``host_block_ids``), staged through pinned memory and copied
    asynchronously. A device tensor is used as is (int64, contiguous); the kernels skip
    negative or too-large entries instead of faulting.
    """
    arr = host_block_ids(block_indices, num_blocks)
    if arr is None:
        return block_indices.contiguous()
    host = torch.from_numpy(arr)
    if device.type == "cuda":
        return host.pin_memory().to(device, non_blocking=True)
    return host


def check_device_block_ids(idx: torch.Tensor, num_blocks: int, what: str) -> None:
    """Strict mode for block tables that live on the device: one ``torch.aminmax`` and one read-back (a device
    synchronisation) before the launch; ``IndexError`` if an id lies outside ``[0, num_blocks)`` — where the
    reference's ``layer_kv[:, idx]`` (elasticmm/engine/v0/worker.py:597, :604) would trip torch's device-side
    assert. Without it the kernels skip such ids (a padded table is legal there) and a caller cannot tell."""
    if idx.numel() == 0:
        return
    lo, hi = (int(x) for x in torch.aminmax(idx))
    if lo < 0 or hi >= num_blocks:
        bad = lo if lo < 0 else hi
        raise IndexError(f"{what}: index {bad} is out of bounds for dimension 1 with size {num_blocks} "
                         f"(device block table, strict mode)")


class PoolView:
    """A block pool as the kernels see it: per-layer base pointers + geometry.

    ``kv_cache`` is the reference's pool: a list of L tensors
    ``[num_kv, num_blocks, block_size, num_heads, head_size]`` (worker.py:388-394,
    :594) or one monolithic tensor ``[L, num_kv, num_blocks, ...]``
    (nccl_transfer.py:215). Trailing dimensions are free (the vision block pool
    ``[num_blocks, tokens, dim]`` is viewed with num_kv = 1).
    """

    def __init__(self, kv_cache: Union[Sequence[torch.Tensor], torch.Tensor], num_kv_dim: bool = True,
                 pinned_host_for: Optional[torch.device] = None):
        """``pinned_host_for``: accept page-locked host tensors (a CPU swap pool) that the
        kernels of the given GPU read and write directly over PCIe."""
        if isinstance(kv_cache, torch.Tensor):
            layers = list(kv_cache.unbind(0))
        else:
            layers = list(kv_cache)
        if not layers:
            raise ValueError("empty KV pool")
        first = layers[0]
        for i, t in enumerate(layers):
            if pinned_host_for is not None:
                if t.is_cuda or not t.is_pinned():
                    raise RuntimeError("PoolView: a host pool must consist of pinned (page-locked) CPU tensors")
            else:
                _require_gpu(t, "PoolView")
            if t.shape != first.shape or t.dtype != first.dtype or t.device != first.device:
                raise ValueError(f"layer {i} differs from layer 0 in shape / dtype / device")
            if not t.is_contiguous():
                raise ValueError(f"layer {i} is not contiguous")
        self.layers: List[torch.Tensor] = layers
        self.device = first.device if pinned_host_for is None else torch.device(pinned_host_for)
        self.on_host = pinned_host_for is not None
        self.dtype = first.dtype
        self.elem_bytes = first.element_size()
        if num_kv_dim:
            self.num_kv = int(first.shape[0])
            self.num_blocks = int(first.shape[1])
            self.block_shape = tuple(first.shape[2:])
        else:
            self.num_kv = 1
            self.num_blocks = int(first.shape[0])
            self.block_shape = tuple(first.shape[1:])
        self.chunk_elems = int(np.prod(self.block_shape, dtype=np.int64)) if self.block_shape else 1
        self.chunk_bytes = self.chunk_elems * self.elem_bytes
        self.ptrs = [t.data_ptr() for t in layers]
        # the host pointer tables the entry points take, built once (the layers stay where they are)
        self._groups = [(l0, ptr_table(self.ptrs[l0:l0 + EMM_MAX_LAYERS]))
                        for l0 in range(0, len(layers), EMM_MAX_LAYERS)]

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def layer_groups(self):
        """(first_layer, ctypes pointer table) per group of at most EMM_MAX_LAYERS layers."""
        return self._groups

    def packed_shape(self, n: int):
        return (self.num_layers, self.num_kv, n) + self.block_shape


def _table_for_launch(block_indices: IndexLike, pool: PoolView, strict: bool, what: str):
    """(n, pointer argument, host?, keep-alive) of a block table for the pack / unpack entry points.

    This sits in front of every launch, and a request of a few dozen blocks is a few microseconds of kernel, so the
    two usual cases are kept short: a contiguous int64 device tensor is passed as it is (trusted, or validated
    when ``strict``), and a short Python list becomes a ctypes array directly (range check with min / max, negative
    ids counted from the end, as torch's indexing does) without a detour through numpy. Everything else goes through
    ``host_block_ids`` / ``block_index_tensor``. Host tables travel in the kernel argument block
    (``*_host_ids`` entry points) unless the pool itself lives in host memory."""
    nb = pool.num_blocks
    if type(block_indices) is torch.Tensor and block_indices.is_cuda:
        idx = block_indices
        if idx.dtype != torch.long:
            raise TypeError(f"block index tensor must be int64, got {idx.dtype}")
        if idx.device != pool.device:  # a table on another GPU: the kernel must not dereference a foreign pointer
            idx = idx.to(pool.device)
        if not idx.is_contiguous():
            idx = idx.contiguous()
        if strict:
            check_device_block_ids(idx, nb, what)
        return idx.numel(), idx.data_ptr(), False, idx
    if type(block_indices) is list and 0 < len(block_indices) <= 64 and not pool.on_host:
        ids = block_indices
        lo, hi = min(ids), max(ids)
        if lo < -nb or hi >= nb:
            raise IndexError(f"index {lo if lo < -nb else hi} is out of bounds for dimension 1 with size {nb}")
        if lo < 0:
            ids = [i + nb if i < 0 else i for i in ids]
        try:
            arr = (_lib.c_int64 * len(ids))(*ids)
            return len(ids), arr, True, arr
        except TypeError:  # not plain Python ints (numpy scalars, nested lists): the general path sorts it out
            pass
    host = host_block_ids(block_indices, nb)
    if host is not None and not pool.on_host:
        return host.size, host.ctypes.data, True, host
    idx = block_index_tensor(host if host is not None else block_indices, nb, pool.device)
    return idx.numel(), idx.data_ptr(), False, idx


def kv_pack(pool: PoolView, block_indices: IndexLike, out: Optional[torch.Tensor] = None,
            strict: bool = False) -> torch.Tensor:
    """Gather ``n`` blocks of every layer into ``[L, num_kv, n, *block_shape]``.

    Host tables (lists, numpy, CPU tensors) are always checked with torch's indexing rules. A DEVICE table is
    trusted: ids outside ``[0, num_blocks)`` are skipped by the kernel and their rows of the result keep whatever
    the allocation held. ``strict=True`` validates a device table first (``check_device_block_ids``: one
    reduction and a synchronisation) and raises ``IndexError`` instead."""
    lib = _lib.load()
    n, table_arg, inline, keep = _table_for_launch(block_indices, pool, strict, "kv_pack")
    if out is None:
        out = torch.empty((pool.num_layers, pool.num_kv, n) + pool.block_shape, dtype=pool.dtype, device=pool.device)
    elif out.device != pool.device or out.dtype != pool.dtype or not out.is_contiguous() \
            or out.numel() != pool.num_layers * pool.num_kv * n * pool.chunk_elems:
        raise ValueError("kv_pack: `out` must be a contiguous pool-dtype tensor of the packed size")
    stream = _stream_ptr(pool.device)
    plane = pool.num_kv * n * pool.chunk_bytes
    fn = lib.emm_kv_pack_host_ids if inline else lib.emm_kv_pack
    base = out.data_ptr()
    for l0, table in pool._groups:
        rc = fn(table, len(table), pool.num_kv, pool.num_blocks, pool.chunk_bytes, table_arg, n, base + l0 * plane, stream)
        if rc:
            check(rc, "emm_kv_pack_host_ids" if inline else "emm_kv_pack")
    del keep
    return out


def kv_unpack(pool: PoolView, block_indices: IndexLike, packed: torch.Tensor, strict: bool = False) -> None:
    """Scatter ``packed`` ``[L, num_kv, n, ...]`` into the pool under ``block_indices`` (``strict``: as in
    ``kv_pack``; without it a device table's out-of-range ids are skipped, their rows dropped)."""
    lib = _lib.load()
    if not packed.is_cuda:
        _require_gpu(packed, "kv_unpack")
    n, table_arg, inline, keep = _table_for_launch(block_indices, pool, strict, "kv_unpack")
    if packed.device != pool.device:
        raise ValueError("kv_unpack: packed buffer is on another device")
    have = packed.numel() * packed.element_size()
    if have != pool.num_layers * pool.num_kv * n * pool.chunk_bytes:
        raise ValueError(f"kv_unpack: packed buffer holds {have} bytes, "
                         f"pool geometry needs {pool.num_layers * pool.num_kv * n * pool.chunk_bytes}")
    if not packed.is_contiguous():
        packed = packed.contiguous()
    stream = _stream_ptr(pool.device)
    plane = pool.num_kv * n * pool.chunk_bytes
    fn = lib.emm_kv_unpack_host_ids if inline else lib.emm_kv_unpack
    base = packed.data_ptr()
    for l0, table in pool._groups:
        rc = fn(table, len(table), pool.num_kv, pool.num_blocks, pool.chunk_bytes, table_arg, n, base + l0 * plane, stream)
        if rc:
            check(rc, "emm_kv_unpack_host_ids" if inline else "emm_kv_unpack")
    del keep


def kv_migrate(src: PoolView, src_indices: IndexLike, dst: PoolView, dst_indices: IndexLike,
               strict: bool = False) -> None:
    """``dst[l][:, dst_idx[j]] = src[l][:, src_idx[j]]`` in one launch, no staging buffer (``strict``: as in
    ``kv_pack``, for either table)."""
    lib = _lib.load()
    if strict:
        for idx, pool, what in ((src_indices, src, "kv_migrate (source table)"), (dst_indices, dst, "kv_migrate (destination table)")):
            if isinstance(idx, torch.Tensor) and idx.is_cuda:
                check_device_block_ids(idx, pool.num_blocks, what)
    if (src.num_layers, src.num_kv, src.chunk_bytes, src.device) != (dst.num_layers, dst.num_kv, dst.chunk_bytes, dst.device):
        raise ValueError("kv_migrate: pools differ in layers / kv / chunk size / device")
    if src.on_host and dst.on_host:
        raise ValueError("kv_migrate: at least one pool must live in GPU memory")
    si = block_index_tensor(src_indices, src.num_blocks, src.device)
    di = block_index_tensor(dst_indices, dst.num_blocks, dst.device)
    if si.numel() != di.numel():
        raise ValueError(f"Block count mismatch: src={si.numel()}, dst={di.numel()}")
    stream = _stream_ptr(src.device)
    for (l0, st), (_, dt) in zip(src.layer_groups(), dst.layer_groups()):
        check(lib.emm_kv_migrate(st, src.num_blocks, dt, dst.num_blocks, len(st), src.num_kv, src.chunk_bytes,
                                 si.data_ptr(), di.data_ptr(), si.numel(), stream), "emm_kv_migrate")


def copy_blocks(pool: PoolView, block_mapping: Union[torch.Tensor, Sequence[Sequence[int]]],
                strict: bool = False) -> None:
    """All layers: ``pool[:, dst] = pool[:, src]`` for the (src, dst) rows of ``block_mapping`` (``strict``: a
    device mapping is validated first, as in ``kv_pack``; without it pairs with an id out of range are skipped)."""
    lib = _lib.load()
    if strict and isinstance(block_mapping, torch.Tensor) and block_mapping.is_cuda:
        check_device_block_ids(block_mapping, pool.num_blocks, "copy_blocks")
    if isinstance(block_mapping, torch.Tensor):
        m = block_mapping
        if m.dtype != torch.long or m.dim() != 2 or m.shape[1] != 2:
            raise ValueError("block_mapping must be an int64 tensor of shape [num_pairs, 2]")
        if not m.is_cuda:
            m = block_index_tensor(m.reshape(-1), pool.num_blocks, pool.device).view(-1, 2)
        m = m.contiguous()
    else:
        arr = np.asarray(block_mapping, dtype=np.int64).reshape(-1, 2)
        m = block_index_tensor(arr.reshape(-1), pool.num_blocks, pool.device).view(-1, 2)
    stream = _stream_ptr(pool.device)
    for _, table in pool.layer_groups():
        check(lib.emm_copy_blocks(table, len(table), pool.num_kv, pool.num_blocks, pool.chunk_bytes,
                                  m.data_ptr(), m.shape[0], stream), "emm_copy_blocks")


def _half_code(dt: torch.dtype, what: str, saturate: bool = False) -> int:
    """src_dtype code of the C ABI; ``saturate`` selects the clamping fp8 mode (EMM_FP8_SATURATE)."""
    flag = EMM_FP8_SATURATE if saturate else 0
    if dt == torch.bfloat16:
        return EMM_DTYPE_BF16 | flag
    if dt == torch.float16:
        return EMM_DTYPE_F16 | flag
    raise TypeError(f"{what}: 16-bit side must be bfloat16 or float16, got {dt}")


def _scales_tensor(scales, num_layers: int, device: torch.device) -> torch.Tensor:
    t = scales if isinstance(scales, torch.Tensor) else torch.tensor(scales, dtype=torch.float32)
    t = t.to(device=device, dtype=torch.float32).reshape(-1).contiguous()
    if t.numel() != num_layers:
        raise ValueError(f"expected {num_layers} per-layer scales, got {t.numel()}")
    return t


def kv_unpack_dequant_fp8(pool: PoolView, block_indices: IndexLike, packed_fp8: torch.Tensor,
                          k_scales, v_scales) -> None:
    """Scatter an fp8-e4m3fn transfer buffer ``[L, 2, n, ...]`` into a bf16/f16 pool,
    ``out = rne16(float(q) * scale)`` with per-layer K and V scales."""
    lib = _lib.load()
    _require_gpu(packed_fp8, "kv_unpack_dequant_fp8")
    if pool.num_kv != 2:
        raise ValueError("kv_unpack_dequant_fp8 needs a [2, num_blocks, ...] pool")
    if packed_fp8.element_size() != 1:
        raise TypeError("packed_fp8 must be a 1-byte tensor (float8_e4m3fn or uint8)")
    code = _half_code(pool.dtype, "kv_unpack_dequant_fp8")
    idx = block_index_tensor(block_indices, pool.num_blocks, pool.device)
    n = idx.numel()
    if packed_fp8.numel() != pool.num_layers * 2 * n * pool.chunk_elems:
        raise ValueError("kv_unpack_dequant_fp8: packed buffer size does not match the pool geometry")
    packed_fp8 = packed_fp8.contiguous()
    ks = _scales_tensor(k_scales, pool.num_layers, pool.device)
    vs = _scales_tensor(v_scales, pool.num_layers, pool.device)
    stream = _stream_ptr(pool.device)
    plane = 2 * n * pool.chunk_elems
    for l0, table in pool.layer_groups():
        check(lib.emm_kv_unpack_dequant_fp8(table, len(table), pool.num_blocks, pool.chunk_elems, idx.data_ptr(), n,
                                            packed_fp8.data_ptr() + l0 * plane, ks.data_ptr() + 4 * l0,
                                            vs.data_ptr() + 4 * l0, code, stream), "emm_kv_unpack_dequant_fp8")


def _row_geometry(x: torch.Tensor, what: str):
    """(num_tokens, row_elems, token_stride_elems) of a [T, ...] tensor whose rows are contiguous."""
    shape = x.shape
    nd = len(shape)
    if nd < 1:
        raise ValueError(f"{what}: expected [num_tokens, ...]")
    T = shape[0]
    if T > 0 and x.is_contiguous():  # the common case, kept short: this runs once per layer and call
        row = x.numel() // T
        return T, row, row
    if nd == 1:
        return T, 1, (x.stride(0) if T > 1 else 1)
    row = 1
    for d in shape[1:]:
        row *= d
    strides = x.stride()
    if T > 0:
        # rows must be dense: walk the trailing dimensions from the innermost outwards
        expect = 1
        for d in range(nd - 1, 0, -1):
            if shape[d] != 1 and strides[d] != expect:
                raise ValueError(f"{what}: rows must be contiguous (only the token dimension may be strided)")
            expect *= shape[d]
    return T, row, (strides[0] if T > 1 else row)


def _cache_slots(cache: torch.Tensor, row_elems: int, what: str) -> int:
    if not cache.is_contiguous():
        raise ValueError(f"{what}: cache plane must be contiguous")
    if row_elems == 0:
        return 0
    n = cache.numel()
    if n % row_elems:
        raise ValueError(f"{what}: cache size is not a multiple of the token row")
    return n // row_elems


def reshape_and_cache(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                      slot_mapping: torch.Tensor, k_scale: Optional[torch.Tensor] = None,
                      v_scale: Optional[torch.Tensor] = None, saturate: bool = False) -> None:
    """Append one layer: ``cache.view(slots, row)[slot_mapping[t]] = cvt(x[t])`` for slots >= 0.

    Same-width caches are copied bit for bit; a 1-byte cache with a 16-bit source
    is quantised to fp8-e4m3fn with ``k_scale`` / ``v_scale`` (one float each):
    ``(x.float() / scale).to(float8_e4m3fn)``, or with ``saturate`` the quotient clamped to
    [-448, 448] first (overflow gives +-448 instead of NaN; never the default)."""
    lib = _lib.load()
    if not (key.is_cuda and value.is_cuda and key_cache.is_cuda and value_cache.is_cuda and slot_mapping.is_cuda):
        raise RuntimeError("reshape_and_cache: every tensor must be on the GPU; the KV kernels run on the GPU only")
    if slot_mapping.dtype != torch.long:
        raise TypeError("slot_mapping must be int64")
    if not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.contiguous()
    T, row, ks = _row_geometry(key, "key")
    Tv, rowv, vs = _row_geometry(value, "value")
    if T != Tv or row != rowv:
        raise ValueError("key and value differ in shape")
    if slot_mapping.numel() < T:
        raise ValueError("slot_mapping is shorter than the token count")
    num_slots = _cache_slots(key_cache, row, "key_cache")
    if _cache_slots(value_cache, row, "value_cache") != num_slots:
        raise ValueError("key_cache and value_cache differ in size")
    stream = _stream_ptr(key.device)
    eb = key.element_size()
    ceb = key_cache.element_size()
    if ceb == eb:
        check(lib.emm_reshape_and_cache(key.data_ptr(), value.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(),
                                        slot_mapping.data_ptr(), T, row * eb, ks * eb, vs * eb, num_slots, stream),
              "emm_reshape_and_cache")
    elif ceb == 1 and eb == 2:
        if k_scale is None or v_scale is None:
            raise ValueError("fp8 cache needs k_scale and v_scale")
        code = _half_code(key.dtype, "reshape_and_cache", saturate)
        k_s = _scales_tensor(k_scale, 1, key.device)
        v_s = _scales_tensor(v_scale, 1, key.device)
        check(lib.emm_reshape_and_cache_fp8(key.data_ptr(), value.data_ptr(), key_cache.data_ptr(),
                                            value_cache.data_ptr(), slot_mapping.data_ptr(), T, row, ks, vs,
                                            num_slots, k_s.data_ptr(), v_s.data_ptr(), code, stream),
              "emm_reshape_and_cache_fp8")
    else:
        raise TypeError(f"unsupported source/cache element sizes {eb}/{ceb}")


def reshape_and_cache_strided(keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                              key_caches: Sequence[torch.Tensor], value_caches: Sequence[torch.Tensor],
                              slot_mapping: torch.Tensor, k_scales=None, v_scales=None, saturate: bool = False) -> None:
    """The flash-layout append for caches that are strided views ``[NB, bs, H, D]`` (stride 1 along D),
    such as a head-major pool ``[NB, H, bs, D]`` seen through ``permute(0, 2, 1, 3)``. Caches of the
    sources' element width are copied bit for bit; 1-byte caches with 16-bit sources are quantised to
    fp8-e4m3fn with the per-layer ``k_scales`` / ``v_scales`` (``saturate``: the clamping mode). One launch
    for all layers given (they must share shapes and strides)."""
    lib = _lib.load()
    L = len(keys)
    if not (len(values) == len(key_caches) == len(value_caches) == L):
        raise ValueError("per-layer lists differ in length")
    if L == 0:
        return
    # layer 0 is checked in full; the other layers must repeat its shapes, strides, dtypes and device (a few tuple
    # comparisons per layer: this runs in front of every launch)
    k, v, kc, vc = keys[0], values[0], key_caches[0], value_caches[0]
    for t in (k, v, kc, vc):
        _require_gpu(t, "reshape_and_cache_strided")
    if k.dim() != 3 or v.shape != k.shape:
        raise ValueError("key and value must be [num_tokens, num_heads, head_size] of one shape")
    T, H, D = (int(x) for x in k.shape)
    if kc.dim() != 4 or tuple(kc.shape[2:]) != (H, D) or vc.shape != kc.shape or vc.stride() != kc.stride():
        raise ValueError("caches must be [num_blocks, block_size, num_heads, head_size] views of one geometry")
    eb = k.element_size()
    ceb = kc.element_size()
    fp8 = ceb == 1 and eb == 2
    if v.element_size() != eb or vc.element_size() != ceb or not (fp8 or ceb == eb):
        raise TypeError(f"unsupported source/cache element sizes {eb}/{ceb}")
    if D > 1 and kc.stride(3) != 1:
        raise ValueError("head rows of the cache must be contiguous")
    _, _, ks = _row_geometry(k, "key")
    _, _, vs = _row_geometry(v, "value")
    NB, bs = int(kc.shape[0]), int(kc.shape[1])
    sb, sp, sh = kc.stride(0), kc.stride(1), kc.stride(2)
    sig = lambda t: (t.shape, t.stride(), t.dtype, t.device)  # noqa: E731
    want = (sig(k), sig(v), sig(kc), sig(vc))
    for l in range(1, L):
        if (sig(keys[l]), sig(values[l]), sig(key_caches[l]), sig(value_caches[l])) != want:
            raise ValueError(f"layer {l}: geometry differs from layer 0")
    slot_mapping = _check_slot_mapping(slot_mapping, T)
    stream = _stream_ptr(keys[0].device)
    if fp8:
        if k_scales is None or v_scales is None:
            raise ValueError("fp8 cache needs k_scales and v_scales")
        code = _half_code(k.dtype, "reshape_and_cache_strided", saturate)
        k_s = _scales_tensor(k_scales, L, k.device)
        v_s = _scales_tensor(v_scales, L, k.device)
    for l0 in range(0, L, EMM_MAX_LAYERS):
        sl = slice(l0, l0 + EMM_MAX_LAYERS)
        n = len(keys[sl])
        tables = (ptr_table([t.data_ptr() for t in keys[sl]]), ptr_table([t.data_ptr() for t in values[sl]]),
                  ptr_table([t.data_ptr() for t in key_caches[sl]]), ptr_table([t.data_ptr() for t in value_caches[sl]]))
        if fp8:
            check(lib.emm_reshape_and_cache_strided_fp8(*tables, n, slot_mapping.data_ptr(), T, H, D, bs, NB, ks, vs,
                                                        sb, sp, sh, k_s.data_ptr() + 4 * l0, v_s.data_ptr() + 4 * l0,
                                                        code, stream), "emm_reshape_and_cache_strided_fp8")
        else:
            check(lib.emm_reshape_and_cache_strided(*tables, n, slot_mapping.data_ptr(), T, H, D * eb, bs, NB, ks * eb,
                                                    vs * eb, sb * eb, sp * eb, sh * eb, stream),
                  "emm_reshape_and_cache_strided")


def _paged_geometry(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor):
    """Checks one layer of a paged-layout append; returns (T, H, D, bs, NB, ks, vs, cache_elem_bytes)."""
    for t in (key, value, key_cache, value_cache):
        _require_gpu(t, "reshape_and_cache_paged")
    if key.dim() != 3 or value.shape != key.shape:
        raise ValueError("key and value must be [num_tokens, num_heads, head_size] of one shape")
    T, H, D = (int(v) for v in key.shape)
    if key_cache.dim() != 5 or value_cache.dim() != 4:
        raise ValueError("key_cache must be [NB, H, D/x, bs, x] and value_cache [NB, H, D, bs]")
    NB, Hc, Dx, bs, x = (int(v) for v in key_cache.shape)
    ceb = key_cache.element_size()
    eb = key.element_size()
    if eb != 2 or value.element_size() != 2 or ceb not in (1, 2) or value_cache.element_size() != ceb:
        raise TypeError(f"unsupported source/cache element sizes {eb}/{ceb}")
    if x != 16 // ceb or Hc != H or Dx * x != D:
        raise ValueError(f"key_cache shape {tuple(key_cache.shape)} does not match H={H}, D={D}, x={16 // ceb}")
    if tuple(value_cache.shape) != (NB, H, D, bs):
        raise ValueError(f"value_cache shape {tuple(value_cache.shape)} does not match key_cache")
    if not key_cache.is_contiguous() or not value_cache.is_contiguous():
        raise ValueError("caches must be contiguous")
    _, _, ks = _row_geometry(key, "key")
    _, _, vs = _row_geometry(value, "value")
    return T, H, D, bs, NB, ks, vs, ceb


def _check_slot_mapping(slot_mapping: torch.Tensor, T: int) -> torch.Tensor:
    if slot_mapping.dtype != torch.long or not slot_mapping.is_cuda:
        raise TypeError("slot_mapping must be an int64 GPU tensor")
    if not slot_mapping.is_contiguous():
        slot_mapping = slot_mapping.contiguous()
    if slot_mapping.numel() < T:
        raise ValueError("slot_mapping is shorter than the token count")
    return slot_mapping


def reshape_and_cache_paged(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor,
                            value_cache: torch.Tensor, slot_mapping: torch.Tensor,
                            k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None,
                            saturate: bool = False) -> None:
    """Append one layer into the paged-attention layout:
    ``key_cache[b, h, d // x, o, d % x] = key[t, h, d]``, ``value_cache[b, h, d, o] = value[t, h, d]``
    with ``b, o = divmod(slot_mapping[t], block_size)``; slots < 0 are skipped.

    key / value are ``[T, H, D]``; key_cache ``[NB, H, D // x, bs, x]`` and value_cache
    ``[NB, H, D, bs]``, contiguous, x = 16 // cache element size. A 1-byte cache with a
    16-bit source is quantised to fp8-e4m3fn with ``k_scale`` / ``v_scale``."""
    lib = _lib.load()
    T, H, D, bs, NB, ks, vs, ceb = _paged_geometry(key, value, key_cache, value_cache)
    slot_mapping = _check_slot_mapping(slot_mapping, T)
    k_ptr = v_ptr = None
    keep = None
    if ceb == 1:
        if k_scale is None or v_scale is None:
            raise ValueError("fp8 cache needs k_scale and v_scale")
        keep = (_scales_tensor(k_scale, 1, key.device), _scales_tensor(v_scale, 1, key.device))
        k_ptr, v_ptr = keep[0].data_ptr(), keep[1].data_ptr()
    code = _half_code(key.dtype, "reshape_and_cache_paged", saturate) if ceb == 1 else 0
    check(lib.emm_reshape_and_cache_paged(key.data_ptr(), value.data_ptr(), key_cache.data_ptr(),
                                          value_cache.data_ptr(), slot_mapping.data_ptr(), T, H, D, bs, NB, ks, vs,
                                          code, ceb, k_ptr, v_ptr, _stream_ptr(key.device)),
          "emm_reshape_and_cache_paged")


class PagedLayeredAppend:
    """The paged-layout append for all layers of one step in a single launch (per group of
    EMM_MAX_LAYERS): tensors validated and pointer tables built once, then one C call per
    ``slot_mapping``. The object keeps the tensors alive."""

    def __init__(self, keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                 key_caches: Sequence[torch.Tensor], value_caches: Sequence[torch.Tensor],
                 k_scales=None, v_scales=None, saturate: bool = False):
        self.lib = _lib.load()
        L = len(keys)
        if not (len(values) == len(key_caches) == len(value_caches) == L):
            raise ValueError("per-layer lists differ in length")
        self.num_layers = L
        self._keep = (list(keys), list(values), list(key_caches), list(value_caches))
        if L == 0:
            return
        self.geom = _paged_geometry(keys[0], values[0], key_caches[0], value_caches[0])
        for l in range(1, L):
            if _paged_geometry(keys[l], values[l], key_caches[l], value_caches[l]) != self.geom:
                raise ValueError(f"layer {l}: geometry differs from layer 0")
        self.device = keys[0].device
        self.fp8 = self.geom[7] == 1
        self.code = 0
        self.k_s = self.v_s = None
        if self.fp8:
            if k_scales is None or v_scales is None:
                raise ValueError("fp8 cache needs k_scales and v_scales")
            self.code = _half_code(keys[0].dtype, "PagedLayeredAppend", saturate)
            self.k_s = _scales_tensor(k_scales, L, self.device)
            self.v_s = _scales_tensor(v_scales, L, self.device)
        self.groups = []
        for l0 in range(0, L, EMM_MAX_LAYERS):
            sl = slice(l0, l0 + EMM_MAX_LAYERS)
            self.groups.append((l0, ptr_table([t.data_ptr() for t in keys[sl]]),
                                ptr_table([t.data_ptr() for t in values[sl]]),
                                ptr_table([t.data_ptr() for t in key_caches[sl]]),
                                ptr_table([t.data_ptr() for t in value_caches[sl]])))

    def __call__(self, slot_mapping: torch.Tensor) -> None:
        if self.num_layers == 0:
            return
        T, H, D, bs, NB, ks, vs, ceb = self.geom
        slot_mapping = _check_slot_mapping(slot_mapping, T)
        stream = _stream_ptr(self.device)
        for l0, kt, vt, kct, vct in self.groups:
            k_ptr = self.k_s.data_ptr() + 4 * l0 if self.fp8 else None
            v_ptr = self.v_s.data_ptr() + 4 * l0 if self.fp8 else None
            check(self.lib.emm_reshape_and_cache_paged_layers(kt, vt, kct, vct, len(kt), slot_mapping.data_ptr(), T, H,
                                                              D, bs, NB, ks, vs, self.code, ceb, k_ptr, v_ptr, stream),
                  "emm_reshape_and_cache_paged_layers")


class LayeredAppend:
    """All layers of one step appended with a single launch (per group of EMM_MAX_LAYERS).

    The per-layer tensors are validated and their pointer tables built once; calling the
    object with a ``slot_mapping`` then costs one C call. The tensors are kept alive by the
    object, which suits a serving loop that reuses its key / value staging buffers (or
    replays a captured HIP graph)."""

    def __init__(self, keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                 key_caches: Sequence[torch.Tensor], value_caches: Sequence[torch.Tensor],
                 k_scales=None, v_scales=None, saturate: bool = False):
        self.lib = _lib.load()
        L = len(keys)
        if not (len(values) == len(key_caches) == len(value_caches) == L):
            raise ValueError("per-layer lists differ in length")
        self.num_layers = L
        self._keep = (list(keys), list(values), list(key_caches), list(value_caches))
        if L == 0:
            return
        for t in (*keys, *values, *key_caches, *value_caches):
            _require_gpu(t, "LayeredAppend")
        T, row, ks = _row_geometry(keys[0], "key")
        _, _, vs = _row_geometry(values[0], "value")
        for l in range(L):
            if _row_geometry(keys[l], "key") != (T, row, ks) or _row_geometry(values[l], "value") != (T, row, vs):
                raise ValueError(f"layer {l}: key/value geometry differs from layer 0")
        num_slots = _cache_slots(key_caches[0], row, "key_cache")
        for l in range(L):
            if _cache_slots(key_caches[l], row, "key_cache") != num_slots or \
                    _cache_slots(value_caches[l], row, "value_cache") != num_slots:
                raise ValueError(f"layer {l}: cache size differs from layer 0")
        self.device = keys[0].device
        self.T, self.row, self.ks, self.vs, self.num_slots = T, row, ks, vs, num_slots
        eb = keys[0].element_size()
        ceb = key_caches[0].element_size()
        self.fp8 = ceb == 1 and eb == 2
        if not self.fp8 and ceb != eb:
            raise TypeError(f"unsupported source/cache element sizes {eb}/{ceb}")
        self.eb = eb
        if self.fp8:
            if k_scales is None or v_scales is None:
                raise ValueError("fp8 cache needs k_scales and v_scales")
            self.code = _half_code(keys[0].dtype, "LayeredAppend", saturate)
            self.k_s = _scales_tensor(k_scales, L, self.device)
            self.v_s = _scales_tensor(v_scales, L, self.device)
        self.groups = []
        for l0 in range(0, L, EMM_MAX_LAYERS):
            sl = slice(l0, l0 + EMM_MAX_LAYERS)
            self.groups.append((l0, ptr_table([t.data_ptr() for t in keys[sl]]),
                                ptr_table([t.data_ptr() for t in values[sl]]),
                                ptr_table([t.data_ptr() for t in key_caches[sl]]),
                                ptr_table([t.data_ptr() for t in value_caches[sl]])))

    def __call__(self, slot_mapping: torch.Tensor) -> None:
        if self.num_layers == 0:
            return
        if slot_mapping.dtype != torch.long or not slot_mapping.is_cuda:
            raise TypeError("slot_mapping must be an int64 GPU tensor")
        if not slot_mapping.is_contiguous():
            slot_mapping = slot_mapping.contiguous()
        if slot_mapping.numel() < self.T:
            raise ValueError("slot_mapping is shorter than the token count")
        stream = _stream_ptr(self.device)
        lib = self.lib
        for l0, kt, vt, kct, vct in self.groups:
            if self.fp8:
                check(lib.emm_reshape_and_cache_fp8_layers(kt, vt, kct, vct, len(kt), slot_mapping.data_ptr(), self.T,
                                                           self.row, self.ks, self.vs, self.num_slots,
                                                           self.k_s.data_ptr() + 4 * l0, self.v_s.data_ptr() + 4 * l0,
                                                           self.code, stream), "emm_reshape_and_cache_fp8_layers")
            else:
                eb = self.eb
                check(lib.emm_reshape_and_cache_layers(kt, vt, kct, vct, len(kt), slot_mapping.data_ptr(), self.T,
                                                       self.row * eb, self.ks * eb, self.vs * eb, self.num_slots,
                                                       stream), "emm_reshape_and_cache_layers")


def reshape_and_cache_layers(keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                             key_caches: Sequence[torch.Tensor], value_caches: Sequence[torch.Tensor],
                             slot_mapping: torch.Tensor, k_scales=None, v_scales=None, saturate: bool = False) -> None:
    """Append all layers of one step in a single launch (per group of EMM_MAX_LAYERS)."""
    LayeredAppend(keys, values, key_caches, value_caches, k_scales, v_scales, saturate)(slot_mapping)


def _launch_concat(lib, ptrs, sizes, out: torch.Tensor, stream) -> None:
    off = 0
    for i0 in range(0, len(ptrs), EMM_MAX_SEGMENTS):
        n = min(EMM_MAX_SEGMENTS, len(ptrs) - i0)
        srcs = (_lib.c_void_p * n)(*ptrs[i0:i0 + n])
        nbytes = (_lib.c_int64 * n)(*sizes[i0:i0 + n])
        check(lib.emm_concat_rows(srcs, nbytes, n, out.data_ptr(), off, stream), "emm_concat_rows")
        off += sum(sizes[i0:i0 + n])


def concat_rows(tensors: Sequence[torch.Tensor], out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``torch.cat(tensors, dim=0)`` of ragged ``[rows_i, ...]`` tensors in one launch per
    EMM_MAX_SEGMENTS segments."""
    lib = _lib.load()
    tensors = list(tensors)
    if not tensors:
        raise ValueError("concat_rows: expected a non-empty list of tensors")
    first = tensors[0]
    _require_gpu(first, "concat_rows")
    tail, dtype, device = first.shape[1:], first.dtype, first.device
    row_bytes = first.element_size()
    for d in tail:
        row_bytes *= int(d)
    # one pass per tensor (the host time of this loop is what a short gather waits for)
    # `alive` holds the contiguous copies made here until the launch has been queued: a copy that
    # is dropped earlier goes back to the caching allocator, and the next copy (or `out`) may be
    # handed the same memory before the kernel has read it.
    ptrs, sizes, rows, alive = [], [], 0, []
    for t in tensors:
        if t.shape[1:] != tail or t.dtype != dtype or t.device != device:
            raise ValueError("concat_rows: tensors differ in trailing shape / dtype / device")
        if not t.is_contiguous():
            t = t.contiguous()
            alive.append(t)
        r = t.shape[0]
        rows += r
        ptrs.append(t.data_ptr())
        sizes.append(r * row_bytes)
    shape = (rows,) + tuple(tail)
    if out is None:
        out = torch.empty(shape, dtype=dtype, device=device)
    elif tuple(out.shape) != shape or out.dtype != dtype or out.device != device or not out.is_contiguous():
        raise ValueError("concat_rows: `out` has the wrong shape / dtype / device or is not contiguous")
    _launch_concat(lib, ptrs, sizes, out, _stream_ptr(device))
    del alive  # queued on the stream the copies were made on: the allocator may reuse them now
    return out


class RowSource:
    """A ``[rows, ...]`` GPU tensor prepared as a segment of ``concat_row_sources``: pointer, byte
    count and shape signature are read once, when the tensor enters a cache, so that a gather of
    many cached tensors costs a few dictionary lookups per tensor on the host instead of a dozen
    tensor attribute reads. The object keeps the (contiguous) tensor alive."""
    __slots__ = ("tensor", "ptr", "nbytes", "rows", "sig")

    def __init__(self, t: torch.Tensor):
        _require_gpu(t, "RowSource")
        if t.dim() < 1:
            raise ValueError("RowSource: expected [rows, ...]")
        if not t.is_contiguous():
            t = t.contiguous()
        self.tensor = t
        self.ptr = t.data_ptr()
        self.nbytes = t.numel() * t.element_size()
        self.rows = int(t.shape[0])
        self.sig = (tuple(t.shape[1:]), t.dtype, t.device)


def concat_row_sources(sources: Sequence[RowSource], out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``concat_rows`` over prepared segments."""
    lib = _lib.load()
    if not sources:
        raise ValueError("concat_row_sources: expected a non-empty list")
    sig = sources[0].sig
    ptrs, sizes, rows = [], [], 0
    for s in sources:
        if s.sig is not sig and s.sig != sig:
            raise ValueError("concat_row_sources: segments differ in trailing shape / dtype / device")
        ptrs.append(s.ptr)
        sizes.append(s.nbytes)
        rows += s.rows
    tail, dtype, device = sig
    shape = (rows,) + tail
    if out is None:
        out = torch.empty(shape, dtype=dtype, device=device)
    elif tuple(out.shape) != shape or out.dtype != dtype or out.device != device or not out.is_contiguous():
        raise ValueError("concat_row_sources: `out` has the wrong shape / dtype / device or is not contiguous")
    _launch_concat(lib, ptrs, sizes, out, _stream_ptr(device))
    return out


def stream_copy(src: torch.Tensor, dst: torch.Tensor) -> None:
    """Plain device copy with the block-move tile engine (benchmark yardstick)."""
    lib = _lib.load()
    _require_gpu(src, "stream_copy")
    nbytes = src.numel() * src.element_size()
    if dst.numel() * dst.element_size() != nbytes or not src.is_contiguous() or not dst.is_contiguous():
        raise ValueError("stream_copy: contiguous tensors of equal byte size required")
    check(lib.emm_stream_copy(src.data_ptr(), dst.data_ptr(), nbytes, _stream_ptr(src.device)), "emm_stream_copy")
