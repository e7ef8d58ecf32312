"""TQ4 decompress operator (signature of src/flashquant/kernels/decompress.py:48-86)."""
from __future__ import annotations

from typing import Optional

import torch

from flashquant_amd.kernels._native import native, require_gpu


def tq4_decompress(
    packed: torch.Tensor,
    norms: torch.Tensor,
    centroids: torch.Tensor,
    dtype: torch.dtype = torch.float16,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Decompress nibble-packed TQ4 to (N, H, D) in ``dtype``; the result stays
    in rotated space with coordinate 2j from the high nibble of byte j."""
    require_gpu(packed, "packed")
    return native().tq4_decompress(packed, norms, centroids, dtype, out)


def tq4_decompress_rotated(
    packed: torch.Tensor,
    norms: torch.Tensor,
    centroids: torch.Tensor,
    rotation: torch.Tensor,
    dtype: torch.dtype = torch.float16,
    out: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """``tq4_decompress`` followed by the rotation back to the original space,
    ``(x.float() @ rotation).to(dtype)``, in one launch: what the serving path
    does when it materialises the cache with ``apply_rotation``
    (src/flashquant/vllm/impl.py:298-316).  ``dtype`` is float16 or bfloat16."""
    require_gpu(packed, "packed")
    return native().tq4_decompress_rotated(packed, norms, centroids, rotation, dtype, out)
