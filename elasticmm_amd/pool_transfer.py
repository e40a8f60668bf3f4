"""Gather / scatter on the legacy monolithic pools of the reference.

``elasticmm/engine/v0/nccl_transfer.py`` keeps the KV pool as ONE tensor
``[layers, 2, blocks, block_size, heads, head_dim]`` (:215) and the vision pool as
``[blocks, embed_tokens, embed_dim]`` (:312); its sender stacks per-block slices
and flattens (:241-247, :329-334), its receiver assigns block by block
(:283-289, :361-364). The functions here produce / consume the same flat
messages with one kernel launch each.
"""
from __future__ import annotations

from typing import Sequence

import torch

from . import kv_ops
from .kv_ops import PoolView


def gather_kv_blocks(kv_cache: torch.Tensor, src_blocks: Sequence[int]) -> torch.Tensor:
    """Flat message ``[L*2*n*bs*H*D]`` of the sender (nccl_transfer.py:241-247)."""
    if kv_cache.dim() != 6:
        raise ValueError("expected a [layers, 2, blocks, block_size, heads, head_dim] pool")
    return kv_ops.kv_pack(PoolView(kv_cache), src_blocks).view(-1)


def scatter_kv_blocks(kv_cache: torch.Tensor, dst_blocks: Sequence[int], kv_data_flat: torch.Tensor) -> torch.Tensor:
    """Write a received flat message into ``dst_blocks``; returns it viewed as
    ``[L, 2, n, bs, H, D]`` like the receiver does (nccl_transfer.py:283-293)."""
    if kv_cache.dim() != 6:
        raise ValueError("expected a [layers, 2, blocks, block_size, heads, head_dim] pool")
    L, num_kv, _, bs, H, D = kv_cache.shape
    n = len(dst_blocks)
    total = L * num_kv * n * bs * H * D
    if kv_data_flat.numel() != total:
        raise ValueError(f"message holds {kv_data_flat.numel()} elements, expected {total}")
    kv_data = kv_data_flat.view(L, num_kv, n, bs, H, D)
    kv_ops.kv_unpack(PoolView(kv_cache), dst_blocks, kv_data)
    return kv_data


def gather_vision_blocks(ve_cache: torch.Tensor, src_blocks: Sequence[int]) -> torch.Tensor:
    """Flat message ``[n*tokens*dim]`` (nccl_transfer.py:329-334)."""
    if ve_cache.dim() != 3:
        raise ValueError("expected a [blocks, embed_tokens, embed_dim] pool")
    return kv_ops.kv_pack(PoolView([ve_cache], num_kv_dim=False), src_blocks).view(-1)


def scatter_vision_blocks(ve_cache: torch.Tensor, dst_blocks: Sequence[int], ve_data_flat: torch.Tensor) -> torch.Tensor:
    """nccl_transfer.py:345-368."""
    if ve_cache.dim() != 3:
        raise ValueError("expected a [blocks, embed_tokens, embed_dim] pool")
    n = len(dst_blocks)
    tokens, dim = ve_cache.shape[1], ve_cache.shape[2]
    if ve_data_flat.numel() != n * tokens * dim:
        raise ValueError(f"message holds {ve_data_flat.numel()} elements, expected {n * tokens * dim}")
    ve_data = ve_data_flat.view(n, tokens, dim)
    kv_ops.kv_unpack(PoolView([ve_cache], num_kv_dim=False), dst_blocks, ve_data)
    return ve_data
