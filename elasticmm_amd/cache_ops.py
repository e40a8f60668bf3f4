"""vLLM-shaped cache operators: ``reshape_and_cache_flash``, ``reshape_and_cache`` and ``copy_blocks``.

The reference reaches both inside vLLM (``vllm>=0.10.1``, V0 engine): the append
from ``model_runner.execute_model`` (elasticmm/engine/v0/worker_steps.py:281, :438)
on the pool bound at elasticmm/engine/v0/worker.py:408-412, and ``copy_blocks``
through ``CacheEngine`` (worker.py:380). The signatures below keep vLLM's argument
order so an attention backend can call them unchanged.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import torch

from . import kv_ops
from .kv_ops import PoolView


def reshape_and_cache_flash(key: torch.Tensor, value: torch.Tensor, key_cache: torch.Tensor,
                            value_cache: torch.Tensor, slot_mapping: torch.Tensor, kv_cache_dtype: str = "auto",
                            k_scale: Optional[torch.Tensor] = None, v_scale: Optional[torch.Tensor] = None) -> None:
    """key, value ``[num_tokens, num_heads, head_size]``; caches
    ``[num_blocks, block_size, num_heads, head_size]`` (contiguous, or for "auto" a strided view with
    contiguous head rows such as a permuted head-major pool); ``slot_mapping`` int64
    ``[num_tokens]`` with -1 for padded tokens. ``kv_cache_dtype`` is "auto" (cache
    dtype == key dtype, bit copy) or "fp8" / "fp8_e4m3" (cache is 1 byte wide and
    is written as ``e4m3fn(float(x) / scale)``)."""
    if kv_cache_dtype == "auto":
        if key_cache.element_size() != key.element_size():
            raise ValueError("kv_cache_dtype='auto' needs a cache of the key's element size")
        if key_cache.is_contiguous() and value_cache.is_contiguous():
            kv_ops.reshape_and_cache(key, value, key_cache, value_cache, slot_mapping)
        else:  # e.g. the head-major pool [NB, H, bs, D] passed as a permuted view
            kv_ops.reshape_and_cache_strided([key], [value], [key_cache], [value_cache], slot_mapping)
    elif kv_cache_dtype in ("fp8", "fp8_e4m3"):
        if key_cache.element_size() != 1:
            raise ValueError("fp8 KV cache must be a 1-byte tensor (float8_e4m3fn or uint8)")
        kv_ops.reshape_and_cache(key, value, key_cache, value_cache, slot_mapping, k_scale, v_scale)
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
    elif kv_cache_dtype in ("fp8", "fp8_e4m3"):
        if key_cache.element_size() != 1:
            raise ValueError("fp8 KV cache must be a 1-byte tensor (float8_e4m3fn or uint8)")
        kv_ops.reshape_and_cache_paged(key, value, key_cache, value_cache, slot_mapping, k_scale, v_scale)
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
    elif kv_cache_dtype in ("fp8", "fp8_e4m3"):
        kv_ops.reshape_and_cache_layers(keys, values, key_caches, value_caches, slot_mapping, k_scales, v_scales)
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
    if kv_cache_dtype in ("fp8", "fp8_e4m3"):
        return kv_ops.LayeredAppend(keys, values, key_caches, value_caches, k_scales, v_scales)
    raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")


def paged_layered_append(keys: Sequence[torch.Tensor], values: Sequence[torch.Tensor],
                         key_caches: Sequence[torch.Tensor], value_caches: Sequence[torch.Tensor],
                         kv_cache_dtype: str = "auto", k_scales=None, v_scales=None) -> kv_ops.PagedLayeredAppend:
    """The prepared whole-step append for the paged-attention layout: ``key_caches[l]`` is
    ``[NB, H, D // x, bs, x]``, ``value_caches[l]`` ``[NB, H, D, bs]``; ``plan(slot_mapping)`` is one launch."""
    if kv_cache_dtype == "auto":
        return kv_ops.PagedLayeredAppend(keys, values, key_caches, value_caches)
    if kv_cache_dtype in ("fp8", "fp8_e4m3"):
        return kv_ops.PagedLayeredAppend(keys, values, key_caches, value_caches, k_scales, v_scales)
    raise ValueError(f"unsupported kv_cache_dtype {kv_cache_dtype!r}")


def copy_blocks(kv_caches: List[torch.Tensor], block_mapping: torch.Tensor) -> None:
    """``kv_caches``: list of ``[2, num_blocks, block_size, H, D]``; ``block_mapping``: int64
    ``[num_pairs, 2]`` of (src, dst). One launch covers every layer, K and V."""
    if len(kv_caches) == 0 or block_mapping.numel() == 0:
        return
    kv_ops.copy_blocks(PoolView(kv_caches), block_mapping)
