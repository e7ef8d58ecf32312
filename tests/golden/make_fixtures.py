"""Writes the small committed fixtures under tests/golden/ from the oracle.

Run from the repository root:  python tests/golden/make_fixtures.py
The fixtures guard against drift of torch / LAPACK between machines; they are
data only (matrix entries, codebook levels, one small compress case).
"""
from __future__ import annotations

import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import tq_oracle as O  # noqa: E402


def main() -> None:
    for seed in (42, 43):
        np.save(os.path.join(HERE, f"rotation_d128_seed{seed}.npy"),
                O.haar_orthogonal(128, seed=seed).numpy())
    books = {}
    for bits in (2, 3, 4):
        c, b = O.lloyd_max_gaussian(128, bits)
        books[str(bits)] = {"centroids": [float(v) for v in c], "boundaries": [float(v) for v in b]}
    with open(os.path.join(HERE, "codebook_d128.json"), "w") as f:
        json.dump(books, f, indent=1)

    # one small compress / decompress case: 6 tokens x 2 heads x 128
    g = torch.Generator().manual_seed(7)
    x = torch.randn(6, 2, 128, generator=g)
    x[:, :, 5] *= 10.0
    r = O.haar_orthogonal(128, 42)
    c, b = O.lloyd_max_gaussian(128, 4)
    packed, norms = O.compress(x, r, b)
    np.savez(os.path.join(HERE, "compress_case_6x2x128.npz"),
             x=x.numpy(), packed=packed.numpy(), norms=norms.numpy(),
             recon=O.decompress(packed, norms, c).numpy())


if __name__ == "__main__":
    main()
