"""Index packing (src/flashquant/core/packing.py:54-98, csrc/core/packing.cpp:48-79) on the GPU."""
from flashquant_amd.kernels.packing import nibble_pack, nibble_unpack, pack_2bit, unpack_2bit

__all__ = ["nibble_pack", "nibble_unpack", "pack_2bit", "unpack_2bit"]
