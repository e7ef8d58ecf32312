"""TurboQuantProd keys (3-bit Lloyd-Max + 1-bit sign sketch of the residual,
src/flashquant/core/quantizer.py:270-370) with TQ4 values, as a paged cache.

The reference defines the quantizer but no packed page for it; the record used
here is this package's own: key nibble = ``sign_bit << 3 | index`` and a token
row ``[K nibbles H*D/2 | K norm H*4 | K residual norm H*4 | V idx H*D/2 | V norm H*4]``."""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from flashquant_amd.kernels._native import native, require_gpu


def prod_page_layout(num_kv_heads: int, head_dim: int) -> Tuple[int, int, int, int, int]:
    """Byte offsets (k_norm, k_gamma, v_idx, v_norm, row_bytes) inside a token row."""
    k_norm = num_kv_heads * (head_dim // 2)
    k_gamma = k_norm + 4 * num_kv_heads
    v_idx = k_gamma + 4 * num_kv_heads
    v_norm = v_idx + num_kv_heads * (head_dim // 2)
    return k_norm, k_gamma, v_idx, v_norm, v_norm + 4 * num_kv_heads


def sketch_in_rotated_space(sketch: torch.Tensor, rotation: torch.Tensor) -> torch.Tensor:
    """S @ R.T in float64, rounded once: the matrix that projects a residual held in
    rotated space (``prod_compress`` takes it so that it is computed once, not per call)."""
    return (sketch.double() @ rotation.double().T).float().contiguous()


def prod_compress(
    x: torch.Tensor,
    rotation: torch.Tensor,
    sketch: torch.Tensor,
    boundaries: torch.Tensor,
    centroids: torch.Tensor,
    *,
    sketch_rot: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """TurboQuantProd.quantize for keys ``x`` (N, H, D) fp16/bf16 with the
    (bits - 1) = 3-bit codebook: returns packed nibbles (N, H, D/2) uint8, norms
    (N, H, 1) and residual norms (N, H, 1) float32."""
    require_gpu(x, "x")
    if sketch_rot is None:
        sketch_rot = sketch_in_rotated_space(sketch.to(x.device), rotation.to(x.device))
    return native().prod_compress(x, rotation, sketch_rot, boundaries, centroids)


def prod_store_rows(
    kv_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    k_packed: torch.Tensor,
    k_norms: torch.Tensor,
    k_gamma: torch.Tensor,
    v_packed: torch.Tensor,
    v_norms: torch.Tensor,
) -> None:
    """Assemble token rows and scatter them into the paged cache (num_blocks,
    block_size, H*(D+12)) at the flat slots of ``slot_mapping`` (device tensors)."""
    require_gpu(kv_cache, "kv_cache")
    n, h, half = k_packed.shape
    k_norm, k_gamma_off, v_idx, v_norm, row_bytes = prod_page_layout(h, 2 * half)
    row = torch.empty(n, row_bytes, dtype=torch.uint8, device=kv_cache.device)
    row[:, :k_norm] = k_packed.reshape(n, -1)
    row[:, k_norm:k_gamma_off] = k_norms.reshape(n, h).contiguous().view(torch.uint8)
    row[:, k_gamma_off:v_idx] = k_gamma.reshape(n, h).contiguous().view(torch.uint8)
    row[:, v_idx:v_norm] = v_packed.reshape(n, -1)
    row[:, v_norm:] = v_norms.reshape(n, h).contiguous().view(torch.uint8)
    kv_cache.view(-1, row_bytes)[slot_mapping.long()] = row


def prod_paged_decode(
    q: torch.Tensor,
    kv_cache: torch.Tensor,
    block_table: torch.Tensor,
    seq_lens: torch.Tensor,
    centroids_k3: torch.Tensor,
    centroids_v: torch.Tensor,
    rotation: torch.Tensor,
    sketch: torch.Tensor,
    num_kv_heads: int,
    head_dim: int,
    block_size: int,
    sm_scale: Optional[float] = None,
    out: Optional[torch.Tensor] = None,
    num_splits: int = 0,
) -> torch.Tensor:
    """Single-token attention of ``q`` (num_seqs, H_Q, D), un-rotated, over
    TurboQuantProd key / TQ4 value pages; scores are the estimator of
    TurboQuantProd.estimate_inner_product.  Output in the original space."""
    require_gpu(q, "q")
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(head_dim)
    return native().prod_paged_decode(
        q, kv_cache, block_table, seq_lens, centroids_k3, centroids_v, rotation, sketch,
        num_kv_heads, head_dim, block_size, sm_scale, out, num_splits,
    )
