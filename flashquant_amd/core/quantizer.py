"""TurboQuantMSE and TurboQuantProd (src/flashquant/core/quantizer.py:60-370).

The matrices are made on the host with the reference's seeds and library calls;
``quantize`` / ``dequantize`` / ``estimate_inner_product`` take GPU tensors and
run the float32 HIP row operators (``fq_mse_quantize``, ``fq_mse_dequantize``,
``fq_mse_residual``, ``fq_project_rows``).  head_dim 64, 128 or 256, up to 4
bits."""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch

from flashquant_amd.core.codebook import Codebook, CodebookRegistry
from flashquant_amd.kernels._native import native, require_gpu

_registry = CodebookRegistry()


def haar_orthogonal(dim: int, seed: int = 42) -> torch.Tensor:
    """Seeded Haar rotation, float32 (dim, dim) on the CPU (quantizer.py:60-85)."""
    return native().haar_orthogonal(dim, seed)


def qjl_matrix(dim: int, seed: int = 42, qjl_dim: Optional[int] = None) -> torch.Tensor:
    """Sketch of TurboQuantProd: Gaussian (qjl_dim, dim) / sqrt(qjl_dim), generator
    seeded with ``seed + 1`` (quantizer.py:264-268)."""
    return native().qjl_matrix(dim, seed, qjl_dim)


def split_rotation(rotation: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(rotation.T[:, 0::2], rotation.T[:, 1::2])``, the operands of ``tq4_compress``."""
    return native().split_rotation(rotation)


class TurboQuantMSE:
    """Rotation + Lloyd-Max scalar quantization (quantizer.py:93-195)."""

    def __init__(self, dim: int, bits: int, *, seed: int = 42) -> None:
        if bits < 1 or bits > 4:
            raise ValueError(f"TurboQuantMSE supports 1 to 4 bits, got {bits}")
        self.dim = dim
        self.bits = bits
        self.codebook: Codebook = _registry.get(dim, bits)
        self.rotation = haar_orthogonal(dim, seed=seed)
        self._on_device = {}

    def _device_state(self, device: torch.device):
        state = self._on_device.get(device)
        if state is None:
            state = (self.rotation.to(device), self.codebook.boundaries.to(device), self.codebook.centroids.to(device))
            self._on_device[device] = state
        return state

    def quantize(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        """``(indices int64 (..., dim), norms float32 (..., 1))``."""
        require_gpu(x, "x")
        rot, bnd, _ = self._device_state(x.device)
        return native().mse_quantize(x, rot, bnd, self.bits)

    def dequantize(self, indices: torch.Tensor, norms: torch.Tensor) -> torch.Tensor:
        """float32 (..., dim) in the original space."""
        require_gpu(indices, "indices")
        rot, _, cen = self._device_state(indices.device)
        return native().mse_dequantize(indices, norms, rot, cen)


class TurboQuantProd:
    """(bits - 1)-bit TurboQuantMSE plus one sign bit of the sketched residual per
    coordinate, for unbiased inner products (quantizer.py:203-370)."""

    def __init__(self, dim: int, bits: int, *, qjl_dim: Optional[int] = None, seed: int = 42) -> None:
        if bits < 2:
            raise ValueError(f"TurboQuantProd requires bits >= 2, got {bits}")
        if qjl_dim is not None and qjl_dim != dim:
            raise ValueError("the GPU sketch kernel takes qjl_dim == dim")
        self.dim = dim
        self.bits = bits
        self.mse_quantizer = TurboQuantMSE(dim, bits - 1, seed=seed)
        self.qjl_dim = dim
        self.qjl_matrix = qjl_matrix(dim, seed, dim)
        self._sketch_on_device = {}

    def _sketch(self, device: torch.device) -> torch.Tensor:
        s = self._sketch_on_device.get(device)
        if s is None:
            s = self.qjl_matrix.to(device)
            self._sketch_on_device[device] = s
        return s

    def quantize(self, x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        """``(indices, norms, qjl_signs (+-1 float32), residual_norms)``."""
        require_gpu(x, "x")
        mse = self.mse_quantizer
        rot, _, cen = mse._device_state(x.device)
        indices, norms = mse.quantize(x)
        residual, residual_norms = native().mse_residual(x, indices, norms, rot, cen)
        signs = native().project_rows(residual, self._sketch(x.device), True)
        return indices, norms, signs, residual_norms

    def dequantize(self, indices, norms, qjl_signs, residual_norms) -> torch.Tensor:
        return self.mse_quantizer.dequantize(indices, norms)

    def estimate_inner_product(self, query, indices, norms, qjl_signs, residual_norms) -> torch.Tensor:
        """``<q, k_mse> + gamma sqrt(pi/2) / m <S q, signs>`` with the reference's
        broadcasting over the leading dimensions (quantizer.py:331-370).  The
        dequantization and the sketch of the query are kernels; the two row-wise
        dot products are broadcast elementwise operations on their results."""
        require_gpu(query, "query")
        k_mse = self.mse_quantizer.dequantize(indices, norms)
        mse_term = (query.float() * k_mse).sum(dim=-1, keepdim=True)
        q_proj = native().project_rows(query, self._sketch(query.device), False)
        correction = (q_proj * qjl_signs).sum(dim=-1, keepdim=True)
        scale = residual_norms * math.sqrt(math.pi / 2.0) / self.qjl_dim
        return mse_term + scale * correction
