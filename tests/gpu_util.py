"""Helpers for the GPU parity tests: seeded inputs, oracle-built paged caches."""
from __future__ import annotations

import torch

from oracle import tq_oracle as O

_BOOKS = {}


def book(dim=128, bits=4, seed=42):
    key = (dim, bits, seed)
    if key not in _BOOKS:
        c, b = O.lloyd_max_gaussian(dim, bits)
        _BOOKS[key] = (c, b, O.haar_orthogonal(dim, seed))
    return _BOOKS[key]


def build_paged_case(lens, hq, hkv, d=128, bs=16, seed=3, dtype=torch.bfloat16, extra_blocks=3,
                     kv_scale=1.0):
    """Random K/V per sequence, compressed by the oracle and scattered into a
    paged cache through a seeded random block table.  Unused slots hold random
    bytes, so reads past a sequence's end would show up in the result."""
    c, b, r = book(d)
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    max_blocks = max(1, (max(lens) + bs - 1) // bs)
    nb = S * max_blocks + extra_blocks
    row = hkv * (d + 8)
    cache = torch.randint(0, 256, (nb, bs, row), dtype=torch.uint8, generator=g)
    # random bytes in the norm slots could decode to NaN/Inf; such slots are never
    # read by a correct kernel, and a wrong read then fails loudly
    table = torch.randperm(nb, generator=g)[: S * max_blocks].reshape(S, max_blocks).int()
    for s, L in enumerate(lens):
        if L == 0:
            continue
        k = torch.randn(L, hkv, d, generator=g) * kv_scale
        v = torch.randn(L, hkv, d, generator=g) * kv_scale
        kp, kn = O.compress(k, r, b)
        vp, vn = O.compress(v, r, b)
        t = torch.arange(L)
        slots = table[s].long()[t // bs] * bs + t % bs
        O.store_rows(cache, slots, kp, kn, vp, vn)
    q = torch.randn(S, hq, d, generator=g).to(dtype)
    return q, cache, table, torch.tensor(lens, dtype=torch.int32)
