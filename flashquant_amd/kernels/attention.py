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


def paged_tq4_prefill(
    q: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    max_seqlen_q: int,
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
    causal: bool = True,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Prefill (or chunked prefill) over the packed paged cache in one launch.

    ``q`` (tokens, H_Q, D) holds the un-rotated queries of all sequences, the
    queries of sequence ``s`` at ``cu_seqlens_q[s]:cu_seqlens_q[s+1]``;
    ``seq_lens[s]`` keys (the new tokens included, already stored) are read
    through ``block_table[s]``.  Replaces the serving backend's rotate /
    decompress-the-cache / ``flash_attn_varlen_func`` / rotate-back sequence
    (src/flashquant/vllm/impl.py:317-336, 470-512), with the arguments that
    call takes: ``cu_seqlens_q``, ``max_seqlen_q``, ``seqused_k`` (here
    ``seq_lens``), ``block_table``, ``softmax_scale``, ``causal``."""
    require_gpu(q, "q")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    return native().paged_tq4_prefill(
        q, cu_seqlens_q, int(max_seqlen_q), kv_cache, block_table, seq_lens, centroids_k, centroids_v, rotation,
        num_kv_heads, head_dim, block_size, sm_scale, causal, out
    )
