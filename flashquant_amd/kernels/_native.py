"""Access to the native module for the operator layer."""
from __future__ import annotations

import torch

from flashquant_amd import load_native


def native():
    return load_native()


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} is on {t.device}; flashquant_amd runs on the GPU only and has no CPU fallback"
        )
