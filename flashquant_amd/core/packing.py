"""Nibble packing (src/flashquant/core/packing.py:54-98) on the GPU."""
from flashquant_amd.kernels.packing import nibble_pack, nibble_unpack

__all__ = ["nibble_pack", "nibble_unpack"]
