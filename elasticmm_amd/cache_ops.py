"""vLLM-shaped cache operators: ``reshape_and_cache_flash``, ``reshape_and_cache``, ``copy_blocks`` and ``swap_blocks``.

The reference reaches both inside vLLM (``vllm>=0.10.1``, V0 engine): the append
from ``model_runner.execute_model`` (elasticmm/engine/v0/worker_steps.py:281, :438)
on the pool bound at elasticmm/engine/v0/worker.py:408-412, and ``copy_blocks``
through ``CacheEngine`` (worker.py:380). The signatures below keep vLLM's argument
order so an attention backend can call them unchanged.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from . import kv_ops
from .kv_ops import PoolView

# kv_cache_dtype strings of the fp8 KV cache. "fp8" / "fp8_e4m3" is the cast torch performs,
# (x.float() / scale).to(torch.float8_e4m3fn): what overflows becomes NaN (0x7F / 0xFF). The "_sat"
# names clamp the quotient to [-448, 448] first, the convention of a cache written by vLLM's own fp8
# kernels (the variants the reference leaves open at elasticmm/engine/v0/worker.py:194); it has to be
# asked for by name.
_FP8_MODES = {"fp8": False, "fp8_e4m3": False, "fp8_sat": True, "fp8_e4m3_sat": True}


def reshape_and_cache_flash(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor,
                            value_cache: torch.Tensor, slot_mapping: torch.Tensor, kv_cache_dtype: str = "auto",
                            k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None) -> None:
    """key, value ``[num_tokens, num_heads, head_size]``; caches
    ``[num_blocks, block_size, num_heads, head_size]`` (contiguous, or a strided view with
    contiguous head rows such as a permuted head-major pool); ``slot_mapping`` int64
    ``[num_tokens]`` with -1 for padded tokens. ``kv_cache_dtype`` is "auto" (cache
    dtype == key dtype, bit copy), "fp8" / "fp8_e4m3" (cache is 1 byte wide and
    is written as ``e4m3fn(float(x) / scale)``, torch's cast) or "fp8_sat" / "fp8_e4m3_sat" (the
    same with the quotient clamped to [-448, 448] first)."""
    if kv_cache_dtype == "auto":
        if key_cache.element_size() != key.element_size():
            raise ValueError("kv_cache_dtype='auto' needs a cache of the key's element size")
        if key_cache.is_contiguous() and value_cache.is_contiguous():
            kv_ops.reshape_and_cache(key, value, key_cache, value_cache, slot_mapping)
        else:  # e.g. the head-major pool [NB, H, bs, D] passed as a permuted view
            kv_ops.reshape_and_cache_strided([key], [value], [key_cache], [value_cache], slot_mapping)
    elif kv_cache_dtype in _FP8_MODES:
        if key_cache.element_size() != 1:
            raise ValueError("fp8 KV cache must be a 1-byte tensor (float8_e4m3fn or uint8)")
        if key_cache.is_contiguous() and value_cache.is_contiguous():
            kv_ops.reshape_and_cache(key, value, key_cache, value_cache, slot_mapping, k_scale, v_scale,
                                     saturate=_FP8_MODES[kv_cache_dtype])
        else:  # an fp8 pool in the head-major layout, passed as a permuted view
            kv_ops.reshape_and_cache_strided([key], [value], [key_cache], [value_cache], slot_mapping, k_scale,
                                             v_scale, saturate=_FP8_MODES[kv_cache_dtype])
    else:
        raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")


def reshape_and_cache(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                      slot_mapping: torch.Tensor, kv_cache_dtype: str = "auto",
                      k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None) -> None:
    """The append of vLLM's PagedAttention backends (its default attention path on ROCm): key, value
    ``[num_tokens, num_heads, head_size]``; key_cache ``[num_blocks, num_heads, head_size // x, block_size, x]``,
    value_cache ``[num_blocks, num_heads, head_size, block_size]``, x = 16 // cache element size."""
    if kv_cache_dtype == "auto":
        if key_cache.element_size() != key.element_size():
            raise ValueError("kv_cache_dtype='auto' needs a cache of the key's element size")
        kv_ops.reshape_and_cache_paged(key, value, key_cache, value_cache, slot_mapping)
    elif kv_cache_dtype in _FP8_MODES:
        if key_cache.element_size() != 1:
            raise ValueError("fp8 KV cache must be a 1-byte tensor (float8_e4m3fn or uint8)")
        kv_ops.reshape_and_cache_paged(key, value, key_cache, value_cache, slot_mapping, k_scale, v_scale,
                                       saturate=_FP8_MODES[kv_cache_dtype])
    else:
        raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")


def reshape_and_cache_flash_layers(keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                                   kv_caches: Sequence[torch.Tensor], slot_mapping: torch.Tensor,
                                   kv_cache_dtype: str = "auto", k_scales=None, v_scales=None) -> None:
    """All layers of a step in one launch. ``kv_caches[l]`` is ``[2, num_blocks, block_size, H, D]``."""
    key_caches = [c[0] for c in kv_caches]
    value_caches = [c[1] for c in kv_caches]
    if kv_cache_dtype == "auto":
        kv_ops.reshape_and_cache_layers(keys, values, key_caches, value_caches, slot_mapping)
    elif kv_cache_dtype in _FP8_MODES:
        kv_ops.reshape_and_cache_layers(keys, values, key_caches, value_caches, slot_mapping, k_scales, v_scales,
                                        saturate=_FP8_MODES[kv_cache_dtype])
    else:
        raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")


def layered_append(keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor], kv_caches: Sequence[torch.Tensor],
                   kv_cache_dtype: str = "auto", k_scales=None, v_scales=None) -> kv_ops.LayeredAppend:
    """A prepared whole-step append over fixed key / value staging tensors: validate once,
    then ``plan(slot_mapping)`` is one C call (and can be captured in a HIP graph)."""
    key_caches = [c[0] for c in kv_caches]
    value_caches = [c[1] for c in kv_caches]
    if kv_cache_dtype == "auto":
        return kv_ops.LayeredAppend(keys, values, key_caches, value_caches)
    if kv_cache_dtype in _FP8_MODES:
        return kv_ops.LayeredAppend(keys, values, key_caches, value_caches, k_scales, v_scales,
                                    saturate=_FP8_MODES[kv_cache_dtype])
    raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")


def paged_layered_append(keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                         key_caches: Sequence[torch.Tensor], value_caches: Sequence[torch.Tensor],
                         kv_cache_dtype: str = "auto", k_scales=None, v_scales=None) -> kv_ops.PagedLayeredAppend:
    """The prepared whole-step append for the paged-attention layout: ``key_caches[l]`` is
    ``[NB, H, D // x, bs, x]``, ``value_caches[l]`` ``[NB, H, D, bs]``; ``plan(slot_mapping)`` is one launch."""
    if kv_cache_dtype == "auto":
        return kv_ops.PagedLayeredAppend(keys, values, key_caches, value_caches)
    if kv_cache_dtype in _FP8_MODES:
        return kv_ops.PagedLayeredAppend(keys, values, key_caches, value_caches, k_scales, v_scales,
                                         saturate=_FP8_MODES[kv_cache_dtype])
    raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")


def copy_blocks(kv_caches: Sequence[torch.Tensor], *args, strict: bool = False) -> None:
    """Both call shapes vLLM has for this operator; one launch covers every layer, K and V.

    ``copy_blocks(kv_caches, block_mapping)`` — the attention-backend form: ``kv_caches`` is the list of
    per-layer ``[2, num_blocks, ...]`` pools, ``block_mapping`` int64 ``[num_pairs, 2]`` of (src, dst).

    ``copy_blocks(key_caches, value_caches, block_mapping)`` — the form of ``vllm._custom_ops.copy_blocks``
    that the backends hand their split pools to: per-layer key caches and value caches ``[num_blocks, ...]``
    whose trailing shapes may differ (``[NB, H, D // x, bs, x]`` and ``[NB, H, D, bs]`` in the paged-attention
    layout) as long as a block has the same number of bytes in both.

    ``strict=True`` validates a device-resident ``block_mapping`` before the launch (``IndexError`` for an id outside
    the pool, at the cost of a synchronisation); by default such pairs are skipped by the kernel."""
    if len(args) == 1:
        (block_mapping,) = args
        if len(kv_caches) == 0 or block_mapping.numel() == 0:
            return
        kv_ops.copy_blocks(PoolView(kv_caches), block_mapping, strict=strict)
        return
    if len(args) != 2:
        raise TypeError("copy_blocks(kv_caches, block_mapping) or copy_blocks(key_caches, value_caches, block_mapping)")
    value_caches, block_mapping = args
    if len(kv_caches) != len(value_caches):
        raise ValueError("key_caches and value_caches differ in length")
    if len(kv_caches) == 0 or block_mapping.numel() == 0:
        return
    planes = [t.view(t.shape[0], -1) for t in list(kv_caches) + list(value_caches)]  # one chunk per block and plane
    kv_ops.copy_blocks(PoolView(planes, num_kv_dim=False), block_mapping, strict=strict)


def swap_blocks(src_kv_cache: torch.Tensor, dst_kv_cache: torch.Tensor, src_to_dst) -> None:
    """vLLM's backend-level ``swap_blocks(src_kv_cache, dst_kv_cache, src_to_dst)`` for one layer: block
    ``src_to_dst[j, 0]`` of ``src_kv_cache`` ``[2, NB_src, ...]`` goes to block ``src_to_dst[j, 1]`` of
    ``dst_kv_cache`` ``[2, NB_dst, ...]``, K and V in one launch. One of the two may be a page-locked host
    tensor (vLLM's ``cpu_cache``): the kernel then reads / writes it over PCIe directly. ``src_to_dst`` is an
    int64 ``[num_pairs, 2]`` tensor (vLLM passes it on the CPU) or a list of pairs. The worker-level form with
    side streams and per-request events is ``KVWorker.swap_blocks`` (elasticmm/engine/v0/worker.py:467-526)."""
    pairs = src_to_dst if isinstance(src_to_dst, torch.Tensor) else torch.as_tensor(list(src_to_dst), dtype=torch.long)
    if pairs.numel() == 0:
        return
    if pairs.dim() != 2 or pairs.shape[1] != 2 or pairs.dtype != torch.long:
        raise ValueError("src_to_dst must be int64 pairs [num_pairs, 2]")
    if not (src_kv_cache.is_cuda or dst_kv_cache.is_cuda):
        raise ValueError("swap_blocks: at least one cache must live in GPU memory")
    gpu = src_kv_cache.device if src_kv_cache.is_cuda else dst_kv_cache.device
    src = PoolView([src_kv_cache], pinned_host_for=None if src_kv_cache.is_cuda else gpu)
    dst = PoolView([dst_kv_cache], pinned_host_for=None if dst_kv_cache.is_cuda else gpu)
    kv_ops.kv_migrate(src, pairs[:, 0].contiguous(), dst, pairs[:, 1].contiguous())


def compute_slot_mapping(block_tables: Sequence[Sequence[int]], context_lens: Sequence[int],
                         query_lens: Sequence[int], block_size: int, pad_to: Optional[int] = None,
                         device: Optional[torch.device] = None) -> torch.Tensor:
    """The ``slot_mapping`` of one step, as vLLM's ``prepare_model_input`` derives it from the block tables the
    reference passes in ``SequenceGroupMetadata.block_tables`` (elasticmm/engine/v0/worker_steps.py:186-218): sequence
    i contributes ``query_lens[i]`` tokens at positions ``context_lens[i] + k``, token at position p lives in slot
    ``block_tables[i][p // block_size] * block_size + p % block_size``. Tokens of one sequence are consecutive, so
    a prompt yields runs of consecutive slots. The result is int64, padded with -1 up to ``pad_to`` (the padded
    entries are skipped by the append kernels), pinned when a GPU ``device`` is given and copied there without
    blocking."""
    if not (len(block_tables) == len(context_lens) == len(query_lens)):
        raise ValueError("block_tables, context_lens and query_lens differ in length")
    total = int(sum(query_lens))
    size = total if pad_to is None else int(pad_to)
    if size < total:
        raise ValueError(f"pad_to={pad_to} is smaller than the {total} tokens of the step")
    gpu = device is not None and torch.device(device).type == "cuda"
    out = torch.empty(size, dtype=torch.long, pin_memory=gpu)
    slots = out.numpy()
    slots[total:] = -1
    pos = 0
    for table, ctx, q in zip(block_tables, context_lens, query_lens):
        if q == 0:
            continue
        p = np.arange(ctx, ctx + q, dtype=np.int64)
        blocks = p // block_size
        if blocks[-1] >= len(table):
            raise IndexError(f"a sequence of {ctx + q} tokens needs {int(blocks[-1]) + 1} blocks, its table has {len(table)}")
        slots[pos:pos + q] = np.asarray(table, dtype=np.int64)[blocks] * block_size + p % block_size
        pos += q
    return out.to(device, non_blocking=True) if device is not None else out
