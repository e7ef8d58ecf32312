"""Shared pytest configuration: markers, import path, seeded inputs."""
from __future__ import annotations

import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(42)


def outlier_rows(n, h, d, seed, dtype=torch.float32, n_out=4, gain=10.0):
    """N(0,1) rows with n_out channels per head scaled by gain (the outlier
    rule of the benchmark configurations)."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(n, h, d, generator=g, dtype=torch.float32)
    for head in range(h):
        ch = torch.randperm(d, generator=g)[:n_out]
        x[:, head, ch] *= gain
    return x.to(dtype)
