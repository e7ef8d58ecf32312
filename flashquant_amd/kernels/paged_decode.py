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
