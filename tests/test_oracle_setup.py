"""Pins the oracle's set-up routines (packing, codebook, rotation) against
the reference's known answers and against what the mathematics fixes."""
from __future__ import annotations

import json
import math
import os

import numpy as np
import pytest
import torch
from scipy import integrate, stats

from oracle import tq_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


# ---- packing: reference known answers -------------------------------------

def test_nibble_known_answers_python_tests():
    # tests/test_packing.py:46-64 of the reference
    for pair, byte in (([0, 15], 0x0F), ([15, 0], 0xF0), ([5, 10], 0x5A)):
        idx = torch.tensor([pair], dtype=torch.long)
        packed = O.nibble_pack(idx)
        assert packed.dtype == torch.uint8 and packed[0, 0].item() == byte
        assert torch.equal(O.nibble_unpack(packed), idx)


def test_nibble_known_answers_cpp_tests():
    # csrc/tests/test_packing.cpp:22-28 of the reference
    idx = torch.tensor([[5, 3, 15, 0, 7, 9]], dtype=torch.long)
    assert O.nibble_pack(idx).tolist() == [[83, 240, 121]]


def test_nibble_all_bytes_brute_force():
    packed = torch.arange(256, dtype=torch.uint8).reshape(1, 256)
    un = O.nibble_unpack(packed)
    for b in range(256):
        assert un[0, 2 * b].item() == b // 16 and un[0, 2 * b + 1].item() == b % 16
    assert torch.equal(O.nibble_pack(un), packed)


@pytest.mark.parametrize("d", [64, 128, 256])
def test_nibble_roundtrip(d):
    idx = torch.randint(0, 16, (4, 8, d), dtype=torch.long)
    p = O.nibble_pack(idx)
    assert p.shape == (4, 8, d // 2)
    assert torch.equal(O.nibble_unpack(p), idx)


def test_nibble_errors():
    # tests/test_packing.py:102-117
    with pytest.raises(ValueError, match="Values > 15"):
        O.nibble_pack(torch.tensor([[16, 0]]))
    with pytest.raises(ValueError, match="even"):
        O.nibble_pack(torch.randint(0, 16, (10, 3)))


def test_2bit_roundtrip_and_layout():
    idx = torch.tensor([[3, 0, 1, 2]])
    assert O.pack_2bit(idx).tolist() == [[0b11000110]]
    idx = torch.randint(0, 4, (32, 128))
    assert torch.equal(O.unpack_2bit(O.pack_2bit(idx)), idx)
    with pytest.raises(ValueError):
        O.pack_2bit(torch.zeros(2, 6, dtype=torch.long))


# ---- codebook ---------------------------------------------------------------

@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_codebook_shape_monotone_symmetric(dim, bits):
    c, b = O.lloyd_max_gaussian(dim, bits)
    n = 1 << bits
    assert c.shape == (n,) and b.shape == (n - 1,) and c.dtype == torch.float32
    assert (c[1:] > c[:-1]).all()
    assert ((b > c[:-1]) & (b < c[1:])).all()
    assert (c + c.flip(0)).abs().max() < 1e-5          # tests/test_codebook.py:60-78
    assert torch.allclose(b, ((c[:-1].double() + c[1:].double()) / 2).float(), atol=1e-7)


@pytest.mark.parametrize("dim,bits", [(128, 4), (128, 3), (64, 4), (256, 2)])
def test_codebook_is_lloyd_fixed_point_by_quadrature(dim, bits):
    """Each centroid must be the mean of N(0, 1/dim) over its cell, with the
    outer cells ending at +-3.5 sigma; checked by numerical integration, which
    shares no formula with the solver.  The solver stops after 200 sweeps, which
    for 16 levels is short of full convergence (outer centroid still moving by
    about 1e-8 per sweep), hence the 2e-5 * sigma allowance."""
    c, b = O.lloyd_max_gaussian(dim, bits)
    sigma = 1.0 / math.sqrt(dim)
    edges = [-3.5 * sigma] + [float(v) for v in b.double()] + [3.5 * sigma]
    rv = stats.norm(scale=sigma)
    for i in range(len(c)):
        num, _ = integrate.quad(lambda t: t * rv.pdf(t), edges[i], edges[i + 1], epsabs=1e-14)
        den, _ = integrate.quad(rv.pdf, edges[i], edges[i + 1], epsabs=1e-14)
        assert abs(num / den - float(c[i])) < 2e-5 * sigma


def test_codebook_textbook_distortion_16_levels():
    """The 16-level Lloyd-Max quantizer of a unit Gaussian has distortion
    0.009497 (Max, 1960).  The +-3.5 sigma truncation moves it only slightly."""
    c, b = O.lloyd_max_gaussian(128, 4)
    sigma = 1.0 / math.sqrt(128)
    cu = (c.double() / sigma).tolist()
    edges = [-np.inf] + (b.double() / sigma).tolist() + [np.inf]
    mse = 0.0
    for i in range(16):
        v, _ = integrate.quad(lambda t: (t - cu[i]) ** 2 * stats.norm.pdf(t), edges[i], edges[i + 1])
        mse += v
    assert abs(mse - 0.009497) < 2e-4
    # outermost level of the optimal unit-variance quantizer is 2.733; cutting
    # the support at 3.5 sigma pulls it inwards by under 0.1
    assert 2.733 - 0.1 < cu[-1] < 2.733


def test_codebook_degenerate_sizes():
    # tests/test_codebook.py:117-137
    c, b = O.lloyd_max_gaussian(128, 0)
    assert c.shape == (1,) and b.shape == (0,)
    with pytest.raises((ValueError, ZeroDivisionError, RuntimeError)):
        O.lloyd_max_gaussian(0, 4)


def test_codebook_matches_committed_fixture():
    with open(os.path.join(GOLDEN, "codebook_d128.json")) as f:
        gold = json.load(f)
    for bits in ("2", "3", "4"):
        c, b = O.lloyd_max_gaussian(128, int(bits))
        assert np.allclose(c.numpy(), np.array(gold[bits]["centroids"], dtype=np.float32), atol=1e-7)
        assert np.allclose(b.numpy(), np.array(gold[bits]["boundaries"], dtype=np.float32), atol=1e-7)


# ---- rotation ---------------------------------------------------------------

@pytest.mark.parametrize("dim", [64, 128, 256])
def test_rotation_orthogonal_deterministic(dim):
    r = O.haar_orthogonal(dim, seed=42)
    assert r.shape == (dim, dim) and r.dtype == torch.float32
    assert torch.allclose(r.T @ r, torch.eye(dim), atol=1e-5)
    assert torch.equal(r, O.haar_orthogonal(dim, seed=42))
    assert not torch.allclose(r, O.haar_orthogonal(dim, seed=99), atol=1e-3)


def test_rotation_sign_rule():
    """Q * sign(diag R) makes the triangular factor's diagonal positive:
    diag(rot.T @ G) > 0 for the Gaussian matrix G of the same seed."""
    g = torch.randn(128, 128, generator=torch.Generator().manual_seed(42), dtype=torch.float32)
    r = O.haar_orthogonal(128, seed=42)
    tri = r.T @ g
    assert (torch.diag(tri) > 0).all()
    assert torch.tril(tri, diagonal=-1).abs().max() < 1e-4


def test_rotation_matches_committed_fixture():
    gold = np.load(os.path.join(GOLDEN, "rotation_d128_seed42.npy"))
    r = O.haar_orthogonal(128, seed=42).numpy()
    # LAPACK builds may differ in the last bits; the matrix itself must not.
    assert np.abs(r - gold).max() < 1e-5


def test_split_rotation_reconstructs():
    r = O.haar_orthogonal(128)
    ev, od = O.split_rotation(r)
    assert ev.shape == (128, 64) and od.shape == (128, 64)
    rec = torch.empty(128, 128)
    rec[:, 0::2], rec[:, 1::2] = ev, od
    assert torch.equal(rec, r.T.contiguous())


def test_qjl_matrix_seed_and_scale():
    s = O.qjl_matrix(128, seed=42)
    g = torch.randn(128, 128, generator=torch.Generator().manual_seed(43), dtype=torch.float32)
    assert torch.equal(s, g / math.sqrt(128))
