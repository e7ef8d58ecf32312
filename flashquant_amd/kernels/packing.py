"""Nibble packing on the GPU (signatures of src/flashquant/core/packing.py:54-98)."""
from __future__ import annotations

import torch

from flashquant_amd.kernels._native import native, require_gpu


def nibble_pack(indices: torch.Tensor) -> torch.Tensor:
    """Pack pairs of 4-bit indices ``(..., D)`` (uint8 / int32 / int64, values in
    [0, 15]) into ``(..., D // 2)`` uint8: high nibble = even index.  Raises
    ValueError for an odd last dimension or an index out of range."""
    require_gpu(indices, "indices")
    if indices.shape[-1] % 2 != 0:
        raise ValueError(f"Last dimension must be even for nibble packing, got {indices.shape[-1]}")
    return native().packing.nibble_pack(indices)


def nibble_unpack(packed: torch.Tensor) -> torch.Tensor:
    """Unpack ``(..., D // 2)`` uint8 into int64 indices ``(..., D)``."""
    require_gpu(packed, "packed")
    return native().packing.nibble_unpack(packed)


def pack_2bit(indices: torch.Tensor) -> torch.Tensor:
    """Pack four 2-bit indices per byte, the first in the top bits
    (csrc/core/packing.cpp:48-64).  Raises ValueError for a last dimension not
    divisible by 4 or an index outside [0, 3]."""
    require_gpu(indices, "indices")
    if indices.shape[-1] % 4 != 0:
        raise ValueError(f"Last dim must be divisible by 4, got {indices.shape[-1]}")
    return native().packing.pack_2bit(indices)


def unpack_2bit(packed: torch.Tensor) -> torch.Tensor:
    """Inverse of ``pack_2bit``: int64 indices ``(..., 4 * bytes)``."""
    require_gpu(packed, "packed")
    return native().packing.unpack_2bit(packed)
