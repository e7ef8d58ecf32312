"""Quantization primitives with the names of the reference's ``flashquant.core``
(src/flashquant/core/__init__.py).  Set-up (codebook, rotation, sketch) runs on
the host in the native module, as it does in the reference; every operator on
vectors runs on the GPU through the HIP kernels and raises for CPU tensors."""
from flashquant_amd.core.codebook import Codebook, CodebookRegistry, get_codebook, solve_lloyd_max
from flashquant_amd.core.compressor import (CompressedKeys, CompressedValues, KeyCompressor,
                                            ValueCompressor)
from flashquant_amd.core.packing import nibble_pack, nibble_unpack
from flashquant_amd.core.quantizer import (TurboQuantMSE, TurboQuantProd, haar_orthogonal, qjl_matrix,
                                           split_rotation)

__all__ = [
    "Codebook", "CodebookRegistry", "get_codebook", "solve_lloyd_max",
    "CompressedKeys", "CompressedValues", "KeyCompressor", "ValueCompressor",
    "nibble_pack", "nibble_unpack",
    "TurboQuantMSE", "TurboQuantProd", "haar_orthogonal", "qjl_matrix", "split_rotation",
]
