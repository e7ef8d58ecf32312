"""Seeded random sweep over shapes that the parametrised tests do not list: head counts and group sizes,
head dimensions, page sizes, ragged and empty sequences, split counts, query / key lengths that straddle
tile boundaries, row counts that straddle compress tiles.  Every case goes through `_C` -> C ABI and is
checked against the oracle with the bars of the parity tests (paged decode / prefill: cpu_reference.py:154-368;
compress / decompress: cpu_reference.py:22-94)."""
from __future__ import annotations

import random

import pytest
import torch

from tests import test_gpu_parity as P
from tests.gpu_util import book
from tests.test_gpu_parity import kernel_option  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu


def _heads(rng):
    d = rng.choice([128, 128, 128, 64, 256])
    hkv = rng.choice([8, 8, 8, 4, 2, 1, 16])
    g = rng.choice([1, 2, 3, 4, 4, 5, 8, 16])
    if d == 256:
        hkv, g = min(hkv, 4), min(g, 4)
    return d, hkv, hkv * g


@pytest.mark.parametrize("case", range(100))
def test_random_paged_decode(case):
    rng = random.Random(9100 + case)
    d, hkv, hq = _heads(rng)
    n_seq = rng.choice([1, 2, 3, 5, 9, 17, 33, 40, 64, 70])
    longest = rng.choice([40, 130, 300, 700, 1500, 3000])
    if n_seq > 17:
        longest = min(longest, 700)
    lens = [rng.randint(0, longest) for _ in range(n_seq)]
    if max(lens) == 0:
        lens[0] = 5
    P._decode_case(lens, hq=hq, hkv=hkv, d=d, bs=rng.choice([8, 16, 16, 32]), dtype=rng.choice([torch.bfloat16, torch.float16]),
                   num_splits=rng.choice([0, 1, 2, 3, 5, 8, 17]), seed=100 + case)


@pytest.mark.parametrize("case", range(80))
def test_random_store_and_decode(case, kernel_option):
    """The serving step (new token stored, then decoded over) on random shapes: the in-launch store where the
    staged kernel runs, the two launches elsewhere."""
    kernel_option("compress_three_terms", True)
    rng = random.Random(9500 + case)
    d = rng.choice([128, 128, 128, 128, 64, 256])
    hkv = rng.choice([8, 8, 8, 16, 24, 4, 2, 1]) if d == 128 else rng.choice([8, 4, 2, 16])
    g = rng.choice([1, 2, 4, 4, 5, 8, 16]) if d != 256 else rng.choice([1, 2, 4])
    n_seq = rng.choice([1, 2, 3, 5, 9, 17, 33])
    longest = rng.choice([40, 130, 300, 700, 1500, 3000])
    if n_seq > 9:
        longest = min(longest, 700)
    lens = [rng.randint(1, longest) for _ in range(n_seq)]
    if rng.random() < 0.3:
        lens[rng.randrange(n_seq)] = 0                      # a sequence with nothing to store (slot -1)
    if max(lens) == 0:
        lens[0] = 7
    P._check_serving_step(lens, hkv * g, hkv, d, rng.choice([8, 16, 16, 32]), rng.choice([torch.bfloat16, torch.float16]),
                          rng.choice([0, 1, 2, 3, 5, 8, 17]), seed=700 + case)


@pytest.mark.parametrize("case", range(40))
def test_random_fused_prefill(case):
    rng = random.Random(9200 + case)
    d, hkv, hq = _heads(rng)
    b = rng.randint(1, 3)
    nkv = rng.choice([rng.randint(1, 330), rng.randint(300, 900)])
    causal = rng.random() < 0.6
    nq = nkv if causal and rng.random() < 0.7 else rng.randint(1, nkv)
    if hq * b * nq > 60000:
        nq = max(1, 60000 // (hq * b))
    P._check_prefill(b, hq, hkv, nq, nkv, rng.choice([torch.bfloat16, torch.float16]), causal, d=d, seed=200 + case)


@pytest.mark.parametrize("case", range(30))
def test_random_paged_prefill(case):
    rng = random.Random(9300 + case)
    d, hkv, hq = _heads(rng)
    n_seq = rng.randint(1, 6)
    kv = [rng.randint(0, rng.choice([260, 260, 900])) for _ in range(n_seq)]
    ql = [rng.randint(0, k) if k else 0 for k in kv]
    if sum(ql) == 0:
        kv[0], ql[0] = max(kv[0], 3), 3
    P._check_paged_prefill(ql, kv, hq=hq, hkv=hkv, bs=rng.choice([8, 16, 16, 32]), dtype=rng.choice([torch.bfloat16, torch.float16]),
                           causal=rng.random() < 0.8, d=d, seed=300 + case)


@pytest.mark.parametrize("case", range(20))
def test_random_compress_and_decompress(case):
    rng = random.Random(9400 + case)
    d = rng.choice([64, 128, 128, 256])
    n, h = rng.choice([1, 3, 31, 63, 64, 65, 127, 129, 500, 2049]), rng.choice([1, 2, 3, 8])
    dtype = rng.choice([torch.bfloat16, torch.float16])
    x = P.outlier_rows(n, h, d, seed=400 + case)
    P._check_compress(x, d, dtype)
    # decompress of arbitrary bytes, bit for bit, and with the rotation back
    c, _, r = book(d)
    g = torch.Generator().manual_seed(500 + case)
    packed = torch.randint(0, 256, (n, h, d // 2), dtype=torch.uint8, generator=g)
    norms = torch.rand(n, h, 1, generator=g) * 30 + 0.01
    for out_dtype in (torch.float16, torch.bfloat16, torch.float32):
        want = P.O.decompress(packed, norms, c).to(out_dtype)
        got = P.K.tq4_decompress(packed.to(P.DEV), norms.to(P.DEV), c.to(P.DEV), out_dtype)
        assert torch.equal(got.cpu().view(torch.uint8), want.view(torch.uint8))
