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
