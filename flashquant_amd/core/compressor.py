"""Key / value compressors over (batch, heads, seq, head_dim) tensors
(src/flashquant/core/compressor.py:34-300): keys through TurboQuantProd with
seed 42, values through TurboQuantMSE with seed 43."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from flashquant_amd.core.quantizer import TurboQuantMSE, TurboQuantProd
from flashquant_amd.kernels._native import native


@dataclass
class CompressedKeys:
    indices: torch.Tensor
    norms: torch.Tensor
    qjl_signs: torch.Tensor
    residual_norms: torch.Tensor
    original_dtype: torch.dtype = torch.float16


@dataclass
class CompressedValues:
    indices: torch.Tensor
    norms: torch.Tensor
    original_dtype: torch.dtype = torch.float16


class KeyCompressor:
    def __init__(self, head_dim: int, bits: int = 4, *, seed: int = 42) -> None:
        self.head_dim = head_dim
        self.bits = bits
        self.quantizer = TurboQuantProd(head_dim, bits, seed=seed)

    def compress(self, keys: torch.Tensor) -> CompressedKeys:
        indices, norms, signs, residual_norms = self.quantizer.quantize(keys)
        return CompressedKeys(indices, norms, signs, residual_norms, keys.dtype)

    def decompress(self, compressed: CompressedKeys) -> torch.Tensor:
        out = self.quantizer.dequantize(compressed.indices, compressed.norms, compressed.qjl_signs,
                                        compressed.residual_norms)
        return out.to(compressed.original_dtype)

    def asymmetric_attention_scores(self, query: torch.Tensor, compressed: CompressedKeys) -> torch.Tensor:
        """Attention logits (batch, heads, q_len, kv_len) from compressed keys with the
        two-stage estimator (compressor.py:151-196), without the reference's
        (batch, heads, q_len, kv_len, dim) expansion: both terms are matrix products
        of per-row quantities (plain library GEMMs on the GPU; the serving path is
        ``kernels.prod_paged_decode``)."""
        qz = self.quantizer
        k_mse = qz.mse_quantizer.dequantize(compressed.indices, compressed.norms)
        q_proj = native().project_rows(query, qz._sketch(query.device), False)
        mse_term = torch.matmul(query.float(), k_mse.transpose(-2, -1))
        scale = compressed.residual_norms.transpose(-2, -1) * (1.2533141373155001 / qz.qjl_dim)   # sqrt(pi/2) / m
        qjl_term = torch.matmul(q_proj, compressed.qjl_signs.transpose(-2, -1)) * scale
        return (mse_term + qjl_term).to(query.dtype)


class ValueCompressor:
    def __init__(self, head_dim: int, bits: int = 4, *, seed: int = 43) -> None:
        self.head_dim = head_dim
        self.bits = bits
        self.quantizer = TurboQuantMSE(head_dim, bits, seed=seed)

    def compress(self, values: torch.Tensor) -> CompressedValues:
        indices, norms = self.quantizer.quantize(values)
        return CompressedValues(indices, norms, values.dtype)

    def decompress(self, compressed: CompressedValues) -> torch.Tensor:
        return self.quantizer.dequantize(compressed.indices, compressed.norms).to(compressed.original_dtype)
