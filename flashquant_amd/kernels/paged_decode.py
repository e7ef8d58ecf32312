"""Split-K paged decode operator (signature of
src/flashquant/kernels/paged_decode.py:55-128)."""
from __future__ import annotations

import math
from typing import Optional

import torch

from flashquant_amd.kernels._native import native, require_gpu


def split_k_paged_decode(
    q: torch.Tensor,
    kv_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    rotation: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
    sm_scale: Optional[float] = None,
    out: Optional[torch.Tensor] = None,
    num_splits: int = 0,
) -> torch.Tensor:
    """Single-token attention of ``q`` (num_seqs, H_Q, D) over the packed paged
    TQ4 cache.  ``q`` is un-rotated and the result is in the original space;
    ``num_splits=0`` lets the library choose the split count."""
    require_gpu(q, "q")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    return native().split_k_paged_decode(
        q, kv_cache, block_table, seq_lens, centroids_k, centroids_v, rotation,
        num_kv_heads, head_dim, block_size, sm_scale, out, num_splits,
    )


def tq4_store_and_decode(
    key: torch.Tensor,
    value: torch.Tensor,
    slot_mapping: torch.Tensor,
    q: torch.Tensor,
    kv_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    rotation: torch.Tensor,
    boundaries: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
    sm_scale: Optional[float] = None,
    out: Optional[torch.Tensor] = None,
    num_splits: int = 0,
    *,
    rotation_T_even: Optional[torch.Tensor] = None,
    rotation_T_odd: Optional[torch.Tensor] = None,
    workspace: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """One decode step of the serving path (src/flashquant/vllm/impl.py:362-394):
    ``key`` / ``value`` (num_seqs, H_KV, D), the step's new token of every
    sequence, are compressed into the cache rows ``slot_mapping`` (num_seqs,)
    names, then ``q`` (num_seqs, H_Q, D) attends over the cache, the new token
    included (``seq_lens`` counts it).  Equivalent to ``tq4_compress_and_store``
    followed by ``split_k_paged_decode``; one launch fewer where the staged
    decode kernel runs."""
    require_gpu(q, "q")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    if rotation_T_even is None or rotation_T_odd is None:
        rot_t = rotation.T.contiguous()
        rotation_T_even = rot_t[:, 0::2].contiguous()
        rotation_T_odd = rot_t[:, 1::2].contiguous()
    return native().tq4_store_and_decode(
        key, value, slot_mapping, rotation_T_even, rotation_T_odd, boundaries, q, kv_cache, block_table, seq_lens,
        centroids_k, centroids_v, rotation, num_kv_heads, head_dim, block_size, sm_scale, out, num_splits, workspace,
    )
