"""Lloyd-Max codebooks (src/flashquant/core/codebook.py:58-290).

The solver is host code in the native library (``fq_lloyd_max_gaussian``): the
model of a rotated unit vector's coordinate is N(0, 1/dim) truncated to
+-3.5 sigma, as in the reference's Python solver."""
from __future__ import annotations

from dataclasses import dataclass
from functools import lru_cache
from typing import Dict, Optional, Tuple

import torch

from flashquant_amd.kernels._native import native


@lru_cache(maxsize=32)
def solve_lloyd_max(dim: int, bits: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """``(centroids (2^bits,), boundaries (2^bits - 1,))`` float32 on the CPU."""
    return native().codebook.solve_lloyd_max(dim, bits)


@dataclass
class Codebook:
    """Levels and cell boundaries for one (dim, bits) (codebook.py:158-197)."""

    centroids: torch.Tensor
    boundaries: torch.Tensor
    bits: int
    dim: int

    def quantize(self, x: torch.Tensor) -> torch.Tensor:
        """Index of the cell of every value: the number of boundaries below it
        (``torch.bucketize`` with right=False).  Values only; vectors go through
        ``TurboQuantMSE.quantize``."""
        return torch.bucketize(x, self.boundaries.to(x.device))

    def dequantize(self, indices: torch.Tensor) -> torch.Tensor:
        return self.centroids.to(indices.device)[indices]


class CodebookRegistry:
    """Solves each (dim, bits) once and keeps one copy per device
    (codebook.py:205-264)."""

    def __init__(self) -> None:
        self._device_cache: Dict[Tuple[int, int, torch.device], Codebook] = {}

    def get(self, dim: int, bits: int, device: Optional[torch.device] = None) -> Codebook:
        device = torch.device("cpu") if device is None else torch.device(device)
        key = (dim, bits, device)
        if key not in self._device_cache:
            c, b = solve_lloyd_max(dim, bits)
            self._device_cache[key] = Codebook(c.to(device), b.to(device), bits, dim)
        return self._device_cache[key]

    def clear(self) -> None:
        self._device_cache.clear()


_default_registry = CodebookRegistry()


def get_codebook(dim: int, bits: int, device: Optional[torch.device] = None) -> Codebook:
    return _default_registry.get(dim, bits, device)
