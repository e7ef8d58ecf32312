"""Fused TQ4 attention operator (signature of
src/flashquant/kernels/attention.py:52-107)."""
from __future__ import annotations

import math
from typing import Optional

import torch

from flashquant_amd.kernels._native import native, require_gpu


def fused_tq_attention(
    q: torch.Tensor,
    k_packed: torch.Tensor,
    k_norms: torch.Tensor,
    v_packed: torch.Tensor,
    v_norms: torch.Tensor,
    centroids_k: torch.Tensor,
    centroids_v: torch.Tensor,
    rotation: torch.Tensor,
    sm_scale: Optional[float] = None,
    is_causal: bool = False,
) -> torch.Tensor:
    """Attention of ``q`` (B, H_Q, N_Q, D), un-rotated, over nibble-packed keys
    and values (B, H_KV, N_KV, D/2) with float32 norms (B, H_KV, N_KV, 1).
    The kernel rotates the query, dequantises K and V tile by tile and rotates
    the result back: the output is in the original space, in ``q.dtype``."""
    require_gpu(q, "q")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(q.shape[-1])
    return native().fused_tq_attention(
        q, k_packed, k_norms, v_packed, v_norms, centroids_k, centroids_v, rotation, sm_scale, is_causal
    )
