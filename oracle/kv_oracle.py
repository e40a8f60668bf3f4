"""CPU oracle of the KV-cache data-movement path — TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module. Nothing under ``elasticmm_amd/`` does: the
product path fails loudly when its HIP library is missing instead of falling
back to anything here.

Three independent statements of every operation live here, so that a mistake in
one (a dropped term, a transposed index, an off-by-one in a stride) shows up as
a disagreement:

``ref_*``    the reference's own torch expressions on CPU tensors, restated from
             the cited lines of /root/reference (advanced indexing + stack,
             indexed assignment). This is "the reference CPU path" that
             ``bench.py`` times next to the GPU number.
``c_*``      ctypes bindings of ``oracle/kv_oracle.c`` (explicit loops + memcpy,
             integer-grid fp8 rounding derived from the format definition).
``brute_*``  pure-Python element loops for tiny shapes.

Pinning (what fixes each function besides its own formula) — see
tests/test_oracle.py:
  pack / unpack / copy_blocks / reshape_and_cache / concat_rows:
      ref_* == c_* == brute_* on seeded tiny inputs; committed golden vectors
      (tests/golden/kv_small.npz); invariants (unpack∘pack restores the selected
      blocks, canary-filled untouched blocks stay untouched, slot = arange(T)
      reduces to a plain reshape, -1 rows leave the cache unchanged).
      The reference holds no golden vectors or tests for this path.
  reshape_and_cache, paged-attention layout: ref_* == c_* == brute_*; identity slots reduce to a
      permute of the reshaped input; for any slot table the result equals the flash-layout append
      (pinned above) followed by a permute of the whole cache; golden vector
      tests/golden/paged_small.npz generated from that second statement. vLLM's own kernel is
      absent: parity unpinned against it.
  fp8 quantise (append): c_quant_fp8 == torch's ``.to(torch.float8_e4m3fn)``
      (the library routine that defines the contract) on all 65 536 bf16 inputs x 6 scales
      and on the explicit known answers 448, 464, 465, 480, -1000, 2^-9, 2^-10,
      2^-10*1.0001, 17, 18, 19, inf (bytes 126,126,127,127,255,1,0,1,88,89,90,127);
      SHA-256 of each sweep committed under tests/golden/.
  fp8 quantise, saturating mode: c_quant_fp8_sat == torch.clamp(x.float() / s, -448, 448)
      .to(torch.float8_e4m3fn) on all 65 536 bf16 and f16 inputs x 6 scales; known answers
      (448, 464, 465, 1e6, inf -> 0x7E; NaN -> 0x7F; the negatives with the sign bit); equal to the
      non-saturating cast wherever that one is not 0x7F / 0xFF.
  fp8 dequantise: exhaustive over 256 bytes x scales against torch
      ``(q.float() * s).to(bfloat16)``; NaN bytes are compared as "is NaN"
      because torch's CPU bf16 cast yields 0xFFFF (vectorised) or 0x7FC0
      (scalar) for NaN depending on the code path taken, while this build fixes
      0x7FC0.
  vLLM's reshape_and_cache_flash / copy_blocks (third-party, vllm>=0.10.1, not
      vendored, absent here): parity unpinned against vLLM's binary; pinned
      against the closed forms above and the reference's call sites.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Optional, Sequence

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libkv_oracle.so")
_lib: Optional[ctypes.CDLL] = None


def build(force: bool = False) -> str:
    """Compile oracle/kv_oracle.c with gcc (a few hundred ms)."""
    import subprocess

    src = os.path.join(_HERE, "kv_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["gcc", "-O2", "-fPIC", "-shared", "-Wall", "-o", _LIB_PATH, src, "-lm"])
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_f32_to_e4m3fn.restype = ctypes.c_uint8
        _lib.orc_f32_to_e4m3fn.argtypes = [ctypes.c_float]
        _lib.orc_e4m3fn_to_f32.restype = ctypes.c_float
        _lib.orc_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        _lib.orc_f32_to_bf16.restype = ctypes.c_uint16
        _lib.orc_f32_to_bf16.argtypes = [ctypes.c_float]
        _lib.orc_f32_to_f16.restype = ctypes.c_uint16
        _lib.orc_f32_to_f16.argtypes = [ctypes.c_float]
    return _lib


# --------------------------------------------------------------------------
# ref_*: the reference's torch expressions (CPU tensors)
# --------------------------------------------------------------------------
def ref_extract_kv_blocks(kv_cache: Sequence[torch.Tensor], block_indices: Sequence[int]) -> torch.Tensor:
    """elasticmm/engine/v0/worker.py:597-608 — per-layer ``layer_kv[:, idx, :, :, :]``
    then ``torch.stack(dim=0)`` -> [L, 2, n, bs, H, D]."""
    idx = torch.as_tensor(list(block_indices), dtype=torch.long, device=kv_cache[0].device)
    return torch.stack([layer_kv[:, idx, :, :, :] for layer_kv in kv_cache], dim=0)


def ref_write_kv_blocks(kv_cache: Sequence[torch.Tensor], block_indices: Sequence[int], kv_data: torch.Tensor) -> None:
    """elasticmm/engine/v0/worker.py:623-633 — ``layer_kv[:, idx, :, :, :] = kv_data[l]``."""
    assert kv_data.shape[2] == len(block_indices), \
        f"Block count mismatch: {kv_data.shape[2]} vs {len(block_indices)}"
    idx = torch.as_tensor(list(block_indices), dtype=torch.long, device=kv_cache[0].device)
    for layer_idx, layer_kv in enumerate(kv_cache):
        layer_kv[:, idx, :, :, :] = kv_data[layer_idx]


def ref_pool6d_gather(kv_cache: torch.Tensor, src_blocks: Sequence[int]) -> torch.Tensor:
    """elasticmm/engine/v0/nccl_transfer.py:241-247 — stack of per-block slices of
    one [L,2,NB,bs,H,D] pool on dim 2, flattened."""
    return torch.stack([kv_cache[:, :, b, :, :, :] for b in src_blocks], dim=2).flatten()


def ref_pool6d_scatter(kv_cache: torch.Tensor, dst_blocks: Sequence[int], flat: torch.Tensor) -> torch.Tensor:
    """elasticmm/engine/v0/nccl_transfer.py:283-289 — view back to 6-D, per-block assign."""
    L, two, _, bs, H, D = kv_cache.shape
    kv_data = flat.view(L, two, len(dst_blocks), bs, H, D)
    for i, b in enumerate(dst_blocks):
        kv_cache[:, :, b, :, :, :] = kv_data[:, :, i, :, :, :]
    return kv_data


def ref_vision_gather(ve_cache: torch.Tensor, src_blocks: Sequence[int]) -> torch.Tensor:
    """elasticmm/engine/v0/nccl_transfer.py:329-334 — stack of [tok, dim] blocks."""
    return torch.stack([ve_cache[b] for b in src_blocks], dim=0)


def ref_vision_scatter(ve_cache: torch.Tensor, dst_blocks: Sequence[int], ve_data: torch.Tensor) -> None:
    """elasticmm/engine/v0/nccl_transfer.py:361-364."""
    for i, b in enumerate(dst_blocks):
        ve_cache[b] = ve_data[i]


def ref_copy_blocks(kv_caches: Sequence[torch.Tensor], block_mapping: torch.Tensor) -> None:
    """vLLM copy_blocks(kv_caches, block_mapping[P,2]) (reached via CacheEngine,
    elasticmm/engine/v0/worker.py:380): every layer, ``cache[:, dst] = cache[:, src]``
    with the sources read before any write."""
    src = block_mapping[:, 0].long()
    dst = block_mapping[:, 1].long()
    for p in kv_caches:
        p[:, dst] = p[:, src]


def ref_reshape_and_cache_flash(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor,
                                value_cache: torch.Tensor, slot_mapping: torch.Tensor,
                                kv_cache_dtype: str = "auto",
                                k_scale: Optional[torch.Tensor] = None,
                                v_scale: Optional[torch.Tensor] = None) -> None:
    """vLLM reshape_and_cache_flash as reached from execute_model
    (elasticmm/engine/v0/worker_steps.py:281, :438): for slot >= 0,
    ``cache.view(NB*bs, H, D)[slot] = cvt(x)``; fp8: ``(x.float()/scale).to(float8_e4m3fn)``."""
    valid = slot_mapping >= 0
    slots = slot_mapping[valid]
    NB, bs, H, D = key_cache.shape
    for x, cache, scale in ((key, key_cache, k_scale), (value, value_cache, v_scale)):
        rows = x[valid]
        if kv_cache_dtype.startswith("fp8"):
            rows = (rows.float() / scale.float().reshape(())).to(torch.float8_e4m3fn)
            cache.view(torch.uint8).view(NB * bs, H, D).index_copy_(0, slots, rows.view(torch.uint8))
        else:
            cache.view(NB * bs, H, D).index_copy_(0, slots, rows)


def ref_reshape_and_cache_paged(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor,
                                value_cache: torch.Tensor, slot_mapping: torch.Tensor,
                                kv_cache_dtype: str = "auto",
                                k_scale: Optional[torch.Tensor] = None,
                                v_scale: Optional[torch.Tensor] = None) -> None:
    """vLLM reshape_and_cache (PagedAttention layout) as torch indexed assignment:
    key_cache [NB, H, D/x, bs, x], value_cache [NB, H, D, bs]; for slot >= 0 with
    b, o = divmod(slot, bs): ``key_cache[b, :, :, o, :] = key[t].view(H, D/x, x)`` and
    ``value_cache[b, :, :, o] = value[t]``. fp8 caches are given as uint8."""
    NB, H, Dx, bs, x = key_cache.shape
    valid = slot_mapping >= 0
    slots = slot_mapping[valid]
    b = torch.div(slots, bs, rounding_mode="floor")
    o = slots - b * bs
    k, v = key[valid], value[valid]
    if kv_cache_dtype.startswith("fp8"):
        k = (k.float() / k_scale.float().reshape(())).to(torch.float8_e4m3fn).view(torch.uint8)
        v = (v.float() / v_scale.float().reshape(())).to(torch.float8_e4m3fn).view(torch.uint8)
    # two index tensors separated by slices: the indexed dimension comes first in the result
    key_cache[b, :, :, o, :] = k.reshape(-1, H, Dx, x)
    value_cache[b, :, :, o] = v


def ref_unpack_dequant_fp8(kv_cache: Sequence[torch.Tensor], block_indices: Sequence[int],
                           packed_fp8: torch.Tensor, k_scales: torch.Tensor, v_scales: torch.Tensor) -> None:
    """Dequantising unpack: ``pool[l][kv, idx] = (q.float() * scale).to(pool dtype)``.
    No reference counterpart (its transfer rejects fp8, worker.py:956-966)."""
    idx = torch.as_tensor(list(block_indices), dtype=torch.long)
    L = len(kv_cache)
    q = packed_fp8.view(torch.float8_e4m3fn).float().reshape((L, 2, len(idx)) + tuple(kv_cache[0].shape[2:]))
    for l, layer_kv in enumerate(kv_cache):
        layer_kv[0, idx] = (q[l, 0] * k_scales[l].float()).to(layer_kv.dtype)
        layer_kv[1, idx] = (q[l, 1] * v_scales[l].float()).to(layer_kv.dtype)


def ref_concat_rows(vision_embeds: Sequence[torch.Tensor]) -> torch.Tensor:
    """elasticmm/engine/v0/worker_steps.py:264-267 — single tensor passes through,
    otherwise ``torch.cat(dim=0)``."""
    if len(vision_embeds) == 1:
        return vision_embeds[0]
    return torch.cat(list(vision_embeds), dim=0)


# --------------------------------------------------------------------------
# c_*: bindings of kv_oracle.c (numpy arrays in, in-place / numpy out)
# --------------------------------------------------------------------------
def _np_bytes(t) -> np.ndarray:
    """A writable uint8 numpy view of a contiguous CPU torch tensor / numpy array."""
    if isinstance(t, torch.Tensor):
        assert t.is_contiguous() and t.device.type == "cpu"
        return t.view(torch.uint8).reshape(-1).numpy() if t.element_size() == 1 else \
            t.reshape(-1).view(torch.uint8).numpy()
    a = np.ascontiguousarray(t)
    return a.reshape(-1).view(np.uint8)


def _ptr(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def _ptr_table(arrs: List[np.ndarray]):
    return (ctypes.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])


def _i64(x) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(x, dtype=np.int64))


def c_kv_pack(layers: Sequence[torch.Tensor], idx, chunk_bytes: Optional[int] = None) -> np.ndarray:
    """Returns the packed buffer as uint8 [L, num_kv, n, chunk_bytes]."""
    views = [_np_bytes(p) for p in layers]
    num_kv, NB = layers[0].shape[0], layers[0].shape[1]
    chunk = chunk_bytes or views[0].size // (num_kv * NB)
    idx = _i64(idx)
    out = np.zeros((len(layers), num_kv, len(idx), chunk), dtype=np.uint8)
    lib().orc_kv_pack(_ptr_table(views), len(views), num_kv, ctypes.c_int64(NB), ctypes.c_int64(chunk),
                      _ptr(idx), ctypes.c_int64(len(idx)), _ptr(out))
    return out


def c_kv_unpack(layers: Sequence[torch.Tensor], idx, packed) -> None:
    views = [_np_bytes(p) for p in layers]
    num_kv, NB = layers[0].shape[0], layers[0].shape[1]
    chunk = views[0].size // (num_kv * NB)
    idx = _i64(idx)
    buf = _np_bytes(packed)
    assert buf.size == len(layers) * num_kv * len(idx) * chunk
    lib().orc_kv_unpack(_ptr_table(views), len(views), num_kv, ctypes.c_int64(NB), ctypes.c_int64(chunk),
                        _ptr(idx), ctypes.c_int64(len(idx)), _ptr(buf))


def c_copy_blocks(layers: Sequence[torch.Tensor], mapping) -> None:
    views = [_np_bytes(p) for p in layers]
    num_kv, NB = layers[0].shape[0], layers[0].shape[1]
    chunk = views[0].size // (num_kv * NB)
    m = _i64(mapping).reshape(-1, 2)
    lib().orc_copy_blocks(_ptr_table(views), len(views), num_kv, ctypes.c_int64(NB), ctypes.c_int64(chunk),
                          _ptr(m), ctypes.c_int64(m.shape[0]))


def c_reshape_and_cache(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor,
                        value_cache: torch.Tensor, slot_mapping) -> None:
    T = key.shape[0]
    row = key[0].numel() * key.element_size() if T else 0
    slots = _i64(slot_mapping)
    num_slots = key_cache.shape[0] * key_cache.shape[1]
    lib().orc_reshape_and_cache(_ptr(_np_bytes(key)), _ptr(_np_bytes(value)), _ptr(_np_bytes(key_cache)),
                                _ptr(_np_bytes(value_cache)), _ptr(slots), ctypes.c_int64(T),
                                ctypes.c_int64(row), ctypes.c_int64(row), ctypes.c_int64(row),
                                ctypes.c_int64(num_slots))


def _dtype_code(dt: torch.dtype) -> int:
    return {torch.bfloat16: 0, torch.float16: 1}[dt]


def c_quant_fp8(x: torch.Tensor, scale: float) -> np.ndarray:
    """e4m3fn(float(x) / scale) for a bf16 / f16 tensor; returns uint8 of x.shape."""
    bits = x.contiguous().view(torch.int16).reshape(-1).numpy().view(np.uint16)
    out = np.empty(bits.size, dtype=np.uint8)
    lib().orc_quant_fp8(_ptr(bits), ctypes.c_int64(bits.size), ctypes.c_float(scale), _dtype_code(x.dtype), _ptr(out))
    return out.reshape(tuple(x.shape))


def c_quant_fp8_sat(x: torch.Tensor, scale: float) -> np.ndarray:
    """Saturating variant: e4m3fn(clamp(float(x) / scale, -448, 448)); returns uint8 of x.shape."""
    bits = x.contiguous().view(torch.int16).reshape(-1).numpy().view(np.uint16)
    out = np.empty(bits.size, dtype=np.uint8)
    lib().orc_quant_fp8_sat(_ptr(bits), ctypes.c_int64(bits.size), ctypes.c_float(scale), _dtype_code(x.dtype),
                            _ptr(out))
    return out.reshape(tuple(x.shape))


def ref_quant_fp8_sat(x: torch.Tensor, scale: float) -> torch.Tensor:
    """The saturating cast as a torch expression (uint8 bit patterns): the quotient clamped to the
    finite range of e4m3fn before the library cast. NaN passes through clamp unchanged."""
    q = x.float() / torch.tensor(scale, dtype=torch.float32)
    return torch.clamp(q, -448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)


def c_dequant_fp8(q: np.ndarray, scale: float, out_dtype: torch.dtype = torch.bfloat16) -> np.ndarray:
    """16-bit RNE of float(q) * scale; returns uint16 bit patterns."""
    q = np.ascontiguousarray(q, dtype=np.uint8)
    out = np.empty(q.size, dtype=np.uint16)
    lib().orc_dequant_fp8(_ptr(q.reshape(-1)), ctypes.c_int64(q.size), ctypes.c_float(scale),
                          _dtype_code(out_dtype), _ptr(out))
    return out.reshape(q.shape)


def c_reshape_and_cache_fp8(key: torch.Tensor, value: torch.Tensor, key_cache_u8: torch.Tensor,
                            value_cache_u8: torch.Tensor, slot_mapping, k_scale: float, v_scale: float) -> None:
    T = key.shape[0]
    row = key[0].numel() if T else 0
    slots = _i64(slot_mapping)
    num_slots = key_cache_u8.shape[0] * key_cache_u8.shape[1]
    lib().orc_reshape_and_cache_fp8(_ptr(_np_bytes(key)), _ptr(_np_bytes(value)), _ptr(_np_bytes(key_cache_u8)),
                                    _ptr(_np_bytes(value_cache_u8)), _ptr(slots), ctypes.c_int64(T),
                                    ctypes.c_int64(row), ctypes.c_int64(row), ctypes.c_int64(row),
                                    ctypes.c_int64(num_slots), ctypes.c_float(k_scale), ctypes.c_float(v_scale),
                                    _dtype_code(key.dtype))


def c_reshape_and_cache_paged(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor,
                              value_cache: torch.Tensor, slot_mapping, k_scale: float = 1.0,
                              v_scale: float = 1.0) -> None:
    T, H, D = key.shape
    NB, _, _, bs, x = key_cache.shape
    slots = _i64(slot_mapping)
    lib().orc_reshape_and_cache_paged(_ptr(_np_bytes(key)), _ptr(_np_bytes(value)), _ptr(_np_bytes(key_cache)),
                                      _ptr(_np_bytes(value_cache)), _ptr(slots), ctypes.c_int64(T), H, D, bs,
                                      ctypes.c_int64(NB), ctypes.c_int64(H * D), ctypes.c_int64(H * D),
                                      _dtype_code(key.dtype), key_cache.element_size(),
                                      ctypes.c_float(k_scale), ctypes.c_float(v_scale))


def c_unpack_dequant_fp8(layers: Sequence[torch.Tensor], idx, packed_u8, k_scales, v_scales) -> None:
    views = [_np_bytes(p) for p in layers]
    NB = layers[0].shape[1]
    chunk_elems = layers[0][0, 0].numel()
    idx = _i64(idx)
    buf = _np_bytes(packed_u8)
    ks = np.ascontiguousarray(np.asarray(k_scales, dtype=np.float32))
    vs = np.ascontiguousarray(np.asarray(v_scales, dtype=np.float32))
    lib().orc_kv_unpack_dequant_fp8(_ptr_table(views), len(views), ctypes.c_int64(NB), ctypes.c_int64(chunk_elems),
                                    _ptr(idx), ctypes.c_int64(len(idx)), _ptr(buf), _ptr(ks), _ptr(vs),
                                    _dtype_code(layers[0].dtype))


def c_concat_rows(segs: Sequence[torch.Tensor]) -> np.ndarray:
    views = [_np_bytes(s) for s in segs]
    nbytes = _i64([v.size for v in views])
    out = np.empty(int(nbytes.sum()), dtype=np.uint8)
    lib().orc_concat_rows(_ptr_table(views), _ptr(nbytes), len(views), _ptr(out))
    return out


# --------------------------------------------------------------------------
# brute_*: element loops for tiny shapes
# --------------------------------------------------------------------------
def brute_pack(kv_cache: Sequence[torch.Tensor], idx: Sequence[int]) -> torch.Tensor:
    L = len(kv_cache)
    two, NB, bs, H, D = kv_cache[0].shape
    out = torch.zeros((L, two, len(idx), bs, H, D), dtype=kv_cache[0].dtype)
    for l in range(L):
        for kv in range(two):
            for j, b in enumerate(idx):
                for s in range(bs):
                    for h in range(H):
                        for d in range(D):
                            out[l, kv, j, s, h, d] = kv_cache[l][kv, b, s, h, d]
    return out


def brute_unpack(kv_cache: Sequence[torch.Tensor], idx: Sequence[int], kv_data: torch.Tensor) -> None:
    L = len(kv_cache)
    two, NB, bs, H, D = kv_cache[0].shape
    for l in range(L):
        for kv in range(two):
            for j, b in enumerate(idx):
                for s in range(bs):
                    for h in range(H):
                        for d in range(D):
                            kv_cache[l][kv, b, s, h, d] = kv_data[l, kv, j, s, h, d]


def brute_reshape_and_cache(key, value, key_cache, value_cache, slot_mapping) -> None:
    NB, bs, H, D = key_cache.shape
    for t, s in enumerate([int(v) for v in slot_mapping]):
        if s < 0:
            continue
        blk, off = s // bs, s % bs
        for h in range(H):
            for d in range(D):
                key_cache[blk, off, h, d] = key[t, h, d]
                value_cache[blk, off, h, d] = value[t, h, d]


def brute_reshape_and_cache_paged(key, value, key_cache, value_cache, slot_mapping) -> None:
    NB, H, Dx, bs, x = key_cache.shape
    for t, s in enumerate([int(v) for v in slot_mapping]):
        if s < 0:
            continue
        blk, off = s // bs, s % bs
        for h in range(H):
            for d in range(Dx * x):
                key_cache[blk, h, d // x, off, d % x] = key[t, h, d]
                value_cache[blk, h, d, off] = value[t, h, d]


def brute_copy_blocks(kv_caches, mapping) -> None:
    snap = [p.clone() for p in kv_caches]
    for p, s0 in zip(kv_caches, snap):
        for s, d in mapping:
            p[:, d] = s0[:, s]
