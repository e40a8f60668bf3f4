"""Gather / scatter on the legacy monolithic pools of the reference.

``elasticmm/engine/v0/nccl_transfer.py`` keeps the KV pool as ONE tensor
``[layers, 2, blocks, block_size, heads, head_dim]`` (:215) and the vision pool as
``[blocks, embed_tokens, embed_dim]`` (:312); its sender stacks per-block slices
and flattens (:241-247, :329-334), its receiver assigns block by block
(:283-289, :361-364). The functions here produce / consume the same flat
messages with one kernel launch each.
"""
from __future__ import annotations

from typing import Any, Dict, List, Optional, Sequence

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


class PoolTransferManager:
    """The sender / receiver halves of ``V0NCCLTransferManager`` (nccl_transfer.py:140-377) over a link object
    with ``send(tensor, src, dst, tag)`` / ``recv(src, dst, tag)`` (``worker.LoopbackLink`` on one device; the
    reference's NCCL group between two). A group is a name for a set of ranks; messages are the reference's:
    one flat tensor per call, tag 0 for KV blocks and tag 1 for vision blocks."""

    def __init__(self, link: Any):
        self.link = link
        self.transfer_groups: Dict[str, Dict[str, int]] = {}
        self.total_transfers = 0
        self.total_bytes_transferred = 0

    def create_transfer_group(self, group_name: str, rank: int, world_size: int, port_offset: int = 0) -> Dict[str, int]:
        group = {"rank": rank, "world_size": world_size}
        self.transfer_groups[group_name] = group
        return group

    def get_group(self, group_name: str) -> Optional[Dict[str, int]]:
        return self.transfer_groups.get(group_name)

    def _group(self, group_name: str) -> Dict[str, int]:
        group = self.get_group(group_name)
        if not group:
            raise ValueError(f"Group '{group_name}' not found")
        return group

    def transfer_kv_cache_blocks_sync(self, group_name: str, src_worker_rank: int, dst_worker_rank: int,
                                      kv_cache: torch.Tensor, src_blocks: List[int], dst_blocks: List[int],
                                      is_sender: bool) -> Optional[torch.Tensor]:
        """nccl_transfer.py:198-293: the sender gathers ``src_blocks`` and sends the flat message (returns
        None); the receiver takes it, writes ``dst_blocks`` and returns the message viewed as
        ``[L, 2, n, bs, H, D]``."""
        self._group(group_name)
        if is_sender:
            flat = gather_kv_blocks(kv_cache, src_blocks)
            self.link.send(flat, src=src_worker_rank, dst=dst_worker_rank, tag=0)
            self.total_transfers += 1
            self.total_bytes_transferred += flat.numel() * flat.element_size()
            return None
        flat = self.link.recv(src=src_worker_rank, dst=dst_worker_rank, tag=0)
        if flat.dtype != kv_cache.dtype:
            raise ValueError(f"message dtype {flat.dtype} differs from the pool's {kv_cache.dtype}")
        return scatter_kv_blocks(kv_cache, dst_blocks, flat)

    def transfer_vision_embeddings_sync(self, group_name: str, src_worker_rank: int, dst_worker_rank: int,
                                        ve_cache: torch.Tensor, src_blocks: List[int], dst_blocks: List[int],
                                        is_sender: bool) -> Optional[torch.Tensor]:
        """nccl_transfer.py:295-368, same two halves on the ``[blocks, embed_tokens, embed_dim]`` pool."""
        self._group(group_name)
        if is_sender:
            self.link.send(gather_vision_blocks(ve_cache, src_blocks), src=src_worker_rank, dst=dst_worker_rank, tag=1)
            return None
        flat = self.link.recv(src=src_worker_rank, dst=dst_worker_rank, tag=1)
        if flat.dtype != ve_cache.dtype:
            raise ValueError(f"message dtype {flat.dtype} differs from the pool's {ve_cache.dtype}")
        return scatter_vision_blocks(ve_cache, dst_blocks, flat)

    async def transfer_kv_cache_blocks(self, group_name: str, src_worker_rank: int, dst_worker_rank: int,
                                       kv_cache: torch.Tensor, src_blocks: List[int], dst_blocks: List[int],
                                       is_sender: bool) -> Optional[torch.Tensor]:
        return self.transfer_kv_cache_blocks_sync(group_name, src_worker_rank, dst_worker_rank, kv_cache, src_blocks,
                                                  dst_blocks, is_sender)

    async def transfer_vision_embeddings(self, group_name: str, src_worker_rank: int, dst_worker_rank: int,
                                         ve_cache: torch.Tensor, src_blocks: List[int], dst_blocks: List[int],
                                         is_sender: bool) -> Optional[torch.Tensor]:
        return self.transfer_vision_embeddings_sync(group_name, src_worker_rank, dst_worker_rank, ve_cache, src_blocks,
                                                    dst_blocks, is_sender)

    def get_stats(self) -> Dict[str, Any]:
        return {
            "total_transfers": self.total_transfers,
            "total_bytes_transferred": self.total_bytes_transferred,
            "total_mb_transferred": self.total_bytes_transferred / (1024 ** 2),
            "num_groups": len(self.transfer_groups),
        }
