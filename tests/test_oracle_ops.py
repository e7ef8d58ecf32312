"""Pins the oracle's operators (compress, decompress, attention, paged decode,
TurboQuantProd) by brute force on tiny inputs, library routines and
invariants, so that a dropped term, wrong sign or transposed operand fails."""
from __future__ import annotations

import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import tq_oracle as O
from tests.conftest import outlier_rows

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


@pytest.fixture(scope="module")
def book():
    c, b = O.lloyd_max_gaussian(128, 4)
    return c, b, O.haar_orthogonal(128, 42)


# ---- compress ---------------------------------------------------------------

def test_compress_tie_rule_and_division():
    """(3,4) has norm 5; the unit vector is (0.6f, 0.8f).  With boundaries
    placed exactly on those values the index counts boundaries strictly below
    the coordinate (torch.bucketize, right=False)."""
    x = torch.tensor([[[3.0, 4.0]]])
    a, b = torch.tensor(3.0) / 5.0, torch.tensor(4.0) / 5.0
    bnd = torch.stack([a, b])
    packed, norms = O.compress(x, torch.eye(2), bnd)
    assert norms.item() == 5.0
    assert packed.tolist() == [[[(0 << 4) | 1]]]
    # a rotation that swaps the coordinates must swap the nibbles: y = x_hat @ R.T
    swap = torch.tensor([[0.0, 1.0], [1.0, 0.0]])
    packed, _ = O.compress(x, swap, bnd)
    assert packed.tolist() == [[[(1 << 4) | 0]]]
    # a non-symmetric rotation tells R.T from R: R = [[0,1],[-1,0]], y = (x1, -x0)
    rot = torch.tensor([[0.0, 1.0], [-1.0, 0.0]])
    packed, _ = O.compress(x, rot, torch.tensor([-0.7, 0.7]))
    assert packed.tolist() == [[[(2 << 4) | 1]]]       # y = (0.8, -0.6)


def test_compress_scalar_brute_force(book):
    c, b, r = book
    x = outlier_rows(3, 2, 128, seed=5)
    packed, norms = O.compress(x, r, b)
    idx = O.nibble_unpack(packed)
    r64, b64 = r.double().tolist(), b.double().tolist()
    for n in range(3):
        for h in range(2):
            row = x[n, h].double().tolist()
            nrm = math.sqrt(sum(v * v for v in row))
            assert abs(nrm - norms[n, h, 0].item()) < 1e-5 * nrm
            for j in range(128):
                y = sum(row[k] / (nrm + 1e-10) * r64[j][k] for k in range(128))
                want = sum(1 for t in b64 if t < y)
                if min(abs(y - t) for t in b64) > 1e-6:
                    assert idx[n, h, j].item() == want, (n, h, j)


def test_compress_adversarial_inputs_stay_in_range(book):
    # the cases of the reference's tests/test_adversarial.py
    c, b, r = book
    for x in (torch.zeros(2, 2, 128), torch.full((2, 2, 128), 1e6),
              torch.full((2, 2, 128), 1e-30)):
        packed, norms = O.compress(x, r, b)
        assert torch.isfinite(norms).all()
        assert torch.isfinite(O.decompress(packed, norms, c)).all()
    x = torch.randn(2, 2, 128)
    x[0, 0, 3] = 1e8
    packed, norms = O.compress(x, r, b)
    assert torch.isfinite(norms).all()


def test_compress_matches_committed_case(book):
    c, b, r = book
    z = np.load(os.path.join(GOLDEN, "compress_case_6x2x128.npz"))
    packed, norms = O.compress(torch.from_numpy(z["x"]), r, b)
    mism = (O.nibble_unpack(packed) != O.nibble_unpack(torch.from_numpy(z["packed"]))).float().mean()
    assert mism <= 1e-3       # 1536 entries: at most one boundary flip across BLAS builds
    assert np.allclose(norms.numpy(), z["norms"], rtol=1e-6)


def test_config0_round_trip_distortion(book):
    """BASELINE configuration 0: one layer, 8 KV heads, d=128, 4096 tokens,
    outlier channels; relative MSE of the 4-bit round trip is the Lloyd-Max
    distortion (about 0.0095) and the record is 68 bytes per token per head."""
    c, b, r = book
    x = outlier_rows(4096, 8, 128, seed=1000)
    packed, norms = O.compress(x, r, b)
    rec = (O.decompress(packed, norms, c).reshape(-1, 128) @ r).reshape(x.shape)
    rel = ((x - rec) ** 2).sum() / (x ** 2).sum()
    assert abs(rel.item() - 0.0095) < 0.001
    assert packed.shape[-1] + norms.shape[-1] * 4 == 68
    cos = F.cosine_similarity(x.reshape(-1, 128), rec.reshape(-1, 128), dim=-1)
    assert cos.min() > 0.93        # tests/test_quantizer_mse.py:37-41


# ---- decompress -------------------------------------------------------------

def test_decompress_brute_force(book):
    c, _, _ = book
    packed = torch.randint(0, 256, (3, 2, 64), dtype=torch.uint8)
    norms = torch.rand(3, 2, 1) * 7
    out = O.decompress(packed, norms, c)
    assert out.shape == (3, 2, 128) and out.dtype == torch.float32
    for n in range(3):
        for h in range(2):
            for j in range(64):
                byte = packed[n, h, j].item()
                assert out[n, h, 2 * j].item() == (c[byte >> 4] * norms[n, h, 0]).item()
                assert out[n, h, 2 * j + 1].item() == (c[byte & 15] * norms[n, h, 0]).item()


# ---- attention --------------------------------------------------------------

@pytest.mark.parametrize("causal", [False, True])
def test_attention_against_sdpa(causal):
    q = torch.randn(2, 8, 12, 64)
    k = torch.randn(2, 2, 12, 64)
    v = torch.randn(2, 2, 12, 64)
    got = O.attention(q, k, v, is_causal=causal)
    want = F.scaled_dot_product_attention(
        q, k.repeat_interleave(4, 1), v.repeat_interleave(4, 1), is_causal=causal)
    assert torch.allclose(got, want, atol=1e-5)


def test_attention_causal_is_top_left_and_dropped_for_one_query():
    q = torch.randn(1, 1, 3, 16)
    k = torch.randn(1, 1, 5, 16)
    v = torch.randn(1, 1, 5, 16)
    got = O.attention(q, k, v, is_causal=True)
    for i in range(3):   # query i sees keys 0..i
        want = O.attention(q[:, :, i:i + 1], k[:, :, :i + 1], v[:, :, :i + 1])
        assert torch.allclose(got[:, :, i:i + 1], want, atol=1e-6)
    one = O.attention(q[:, :, :1], k, v, is_causal=True)
    assert torch.allclose(one, O.attention(q[:, :, :1], k, v, is_causal=False))


def test_fused_attention_equals_attention_on_reconstruction(book):
    """Rotated-space attention on decompressed K/V, rotated back, equals plain
    attention on the reconstructed K/V in the original space
    (tests/test_attention_kernel.py:95-148 of the reference)."""
    c, b, r = book
    B, HQ, HKV, N = 1, 4, 2, 40
    q = torch.randn(B, HQ, N, 128)
    k = torch.randn(B * HKV * N, 1, 128)
    v = torch.randn(B * HKV * N, 1, 128)
    kp, kn = O.compress(k, r, b)
    vp, vn = O.compress(v, r, b)
    shp = (B, HKV, N)
    got = O.fused_tq_attention(q, kp.reshape(*shp, 64), kn.reshape(*shp, 1), vp.reshape(*shp, 64),
                               vn.reshape(*shp, 1), c, c, r, is_causal=True)
    k_rec = (O.decompress(kp, kn, c).reshape(-1, 128) @ r).reshape(B, HKV, N, 128)
    v_rec = (O.decompress(vp, vn, c).reshape(-1, 128) @ r).reshape(B, HKV, N, 128)
    want = O.attention(q, k_rec, v_rec, is_causal=True)
    assert torch.allclose(got, want, atol=2e-5)


# ---- paged decode -----------------------------------------------------------

def _paged_case(book, lens, hq=8, hkv=2, bs=16, seed=3, dtype=torch.bfloat16):
    c, b, r = book
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    max_blocks = max(1, (max(lens) + bs - 1) // bs)
    nb = S * max_blocks + 3
    cache = torch.randint(0, 256, (nb, bs, hkv * 136), dtype=torch.uint8, generator=g)
    perm = torch.randperm(nb, generator=g)[: S * max_blocks].reshape(S, max_blocks).int()
    for s, L in enumerate(lens):
        if L == 0:
            continue
        k = torch.randn(L, hkv, 128, generator=g)
        v = torch.randn(L, hkv, 128, generator=g)
        kp, kn = O.compress(k, r, b)
        vp, vn = O.compress(v, r, b)
        t = torch.arange(L)
        slots = perm[s].long()[t // bs] * bs + t % bs
        O.store_rows(cache, slots, kp, kn, vp, vn)
    q = torch.randn(S, hq, 128, generator=g).to(dtype)
    return q, cache, perm, torch.tensor(lens, dtype=torch.int32)


def test_page_layout_offsets():
    # src/flashquant/vllm/impl.py:132-138 with 8 heads, d=128
    assert O.page_layout(8, 128) == (512, 544, 1056, 1088)


def test_paged_loop_equals_gather_and_sdpa(book):
    c, b, r = book
    q, cache, bt, lens = _paged_case(book, [37, 0, 16, 5])
    a = O.paged_decode_loop(q, cache, bt, lens, c, c, 2, 128, 16)
    g = O.paged_decode_gather(q, cache, bt, lens, c, c, 2, 128, 16)
    assert torch.equal(a, g)
    assert (a[1] == 0).all()                         # cpu_reference.py:286-287
    k, v = O.gather_sequence(cache, bt[0], 37, c, c, 2, 128, 16)
    want = F.scaled_dot_product_attention(
        q[0].float().unsqueeze(1), k.repeat_interleave(4, 0), v.repeat_interleave(4, 0))
    assert torch.allclose(a[0].float(), want.squeeze(1), atol=2e-2)


def test_paged_block_table_permutation_invariance(book):
    """Moving pages and updating the table must not change the result
    (tests/test_paged_decode_kernel.py:210-259 of the reference)."""
    c, b, r = book
    q, cache, bt, lens = _paged_case(book, [45, 20])
    base = O.split_k_paged_decode(q, cache, bt, lens, c, c, r, 2, 128, 16)
    perm = torch.randperm(cache.shape[0])
    moved = torch.empty_like(cache)
    moved[perm] = cache
    bt2 = perm[bt.long()].int()
    again = O.split_k_paged_decode(q, moved, bt2, lens, c, c, r, 2, 128, 16)
    assert torch.equal(base, again)
    loop = O.split_k_paged_decode(q, cache, bt, lens, c, c, r, 2, 128, 16, faithful_loop=True)
    assert torch.equal(base, loop)


# ---- paged prefill ----------------------------------------------------------

def test_paged_prefill_one_query_is_paged_decode(book):
    c, b, r = book
    q, cache, bt, lens = _paged_case(book, [37, 16, 5])
    cu = torch.arange(4, dtype=torch.int32)
    got = O.paged_prefill(q, cu, cache, bt, lens, c, c, r, 2, 128, 16)
    want = O.split_k_paged_decode(q, cache, bt, lens, c, c, r, 2, 128, 16)
    assert torch.allclose(got.float(), want.float(), atol=1e-2)


def test_paged_prefill_full_queries_is_fused_attention(book):
    """Every token of a sequence is a query: the same numbers as the fused
    operator on that sequence's packed K/V, causal from the top-left corner."""
    c, b, r = book
    hkv, hq, bs, L = 2, 4, 16, 40
    q1, cache, bt, lens = _paged_case(book, [L], hq=hq, hkv=hkv, bs=bs, dtype=torch.float32)
    g = torch.Generator().manual_seed(11)
    q = torch.randn(L, hq, 128, generator=g)
    cu = torch.tensor([0, L], dtype=torch.int32)
    got = O.paged_prefill(q, cu, cache, bt, lens, c, c, r, hkv, 128, bs)
    t = torch.arange(L)
    rows = cache.view(-1, hkv * 136)[bt[0].long()[t // bs] * bs + t % bs]
    kp = rows[:, :hkv * 64].reshape(L, hkv, 64).permute(1, 0, 2)[None]
    kn = rows[:, hkv * 64:hkv * 68].contiguous().view(torch.float32).reshape(L, hkv, 1).permute(1, 0, 2)[None]
    vp = rows[:, hkv * 68:hkv * 132].reshape(L, hkv, 64).permute(1, 0, 2)[None]
    vn = rows[:, hkv * 132:].contiguous().view(torch.float32).reshape(L, hkv, 1).permute(1, 0, 2)[None]
    want = O.fused_tq_attention(q.permute(1, 0, 2)[None], kp, kn, vp, vn, c, c, r, is_causal=True)
    assert torch.allclose(got, want[0].permute(1, 0, 2), atol=2e-5)


def test_paged_prefill_chunk_mask_is_bottom_right(book):
    """A chunked prefill: 7 new tokens on a context of 45.  Checked against
    SDPA with the mask written out by hand, and against the full prefill of
    the same sequence, whose last 7 rows it must reproduce."""
    c, b, r = book
    hkv, hq, bs, L, n = 2, 4, 16, 45, 7
    _, cache, bt, lens = _paged_case(book, [L], hq=hq, hkv=hkv, bs=bs, dtype=torch.float32)
    g = torch.Generator().manual_seed(12)
    q_all = torch.randn(L, hq, 128, generator=g)
    full = O.paged_prefill(q_all, torch.tensor([0, L], dtype=torch.int32), cache, bt, lens, c, c, r, hkv, 128, bs)
    part = O.paged_prefill(q_all[L - n:], torch.tensor([0, n], dtype=torch.int32), cache, bt, lens, c, c, r,
                           hkv, 128, bs)
    assert torch.allclose(part, full[L - n:], atol=1e-6)
    k, v = O.gather_sequence(cache, bt[0], L, c, c, hkv, 128, bs)
    mask = torch.zeros(n, L, dtype=torch.bool)
    for j in range(n):
        mask[j, : L - n + j + 1] = True
    q_rot = (q_all[L - n:] @ r.T).permute(1, 0, 2)
    want = F.scaled_dot_product_attention(q_rot, k.repeat_interleave(2, 0), v.repeat_interleave(2, 0), attn_mask=mask)
    assert torch.allclose(part, want.permute(1, 0, 2) @ r, atol=2e-5)
    no_mask = O.paged_prefill(q_all[L - n:], torch.tensor([0, n], dtype=torch.int32), cache, bt, lens, c, c, r,
                              hkv, 128, bs, causal=False)
    assert not torch.allclose(no_mask[:-1], part[:-1], atol=1e-3)
    assert torch.allclose(no_mask[-1], part[-1], atol=1e-6)     # the last query sees every key either way


# ---- TurboQuantProd ---------------------------------------------------------

def test_prod_signs_and_shapes():
    c3, b3 = O.lloyd_max_gaussian(128, 3)
    r, s = O.haar_orthogonal(128, 42), O.qjl_matrix(128, 42)
    x = torch.randn(5, 128)
    idx, norms, signs, gamma = O.prod_quantize(x, r, b3, c3, s)
    assert idx.max() <= 7 and idx.min() >= 0
    assert set(signs.unique().tolist()) <= {-1.0, 1.0}
    resid = x - O.mse_dequantize(idx, norms, r, c3)
    assert torch.allclose(gamma, resid.norm(dim=-1, keepdim=True))
    assert torch.equal(signs, torch.where(resid @ s.T >= 0, 1.0, -1.0))
    z = O.prod_quantize(torch.zeros(1, 128), r, b3, c3, s)
    assert (z[2] == 1.0).all()      # a zero projection maps to +1


def test_prod_estimator_unbiased():
    """Averaged over many keys the QJL-corrected estimate matches the true
    inner product far better than the MSE-only term
    (tests/test_quantizer_prod.py:32-99 of the reference: relative bias < 0.05)."""
    c3, b3 = O.lloyd_max_gaussian(128, 3)
    r, s = O.haar_orthogonal(128, 42), O.qjl_matrix(128, 42)
    g = torch.Generator().manual_seed(11)
    q = torch.randn(1, 128, generator=g)
    k = q * 0.5 + torch.randn(10000, 128, generator=g)
    idx, norms, signs, gamma = O.prod_quantize(k, r, b3, c3, s)
    est = O.prod_inner_product(q.expand(10000, 128), idx, norms, signs, gamma, r, c3, s).squeeze(-1)
    true = (k * q).sum(-1)
    assert abs((est - true).mean().item()) / true.abs().mean().item() < 0.05
    mse_only = (q * O.mse_dequantize(idx, norms, r, c3)).sum(-1)
    assert abs((est - true).mean()) < abs((mse_only - true).mean()) + 0.05


def test_prod_sketch_term_closed_form_with_identity_sketch():
    """The sketch term by hand.  With S = I (m = d) the stored signs are sign(residual) and
    S q = q, so for q = sign(residual) the sum <S q, signs> is d and the estimate is
    <q, k_mse> + |residual| * sqrt(pi/2) exactly; for q = e_j it is
    <q, k_mse> + |residual| * sqrt(pi/2) / d * sign(residual_j)
    (src/flashquant/core/quantizer.py:355-370).  A dropped, halved or doubled term, a missing
    1/m or a missing residual norm fails this."""
    d = 128
    c3, b3 = O.lloyd_max_gaussian(d, 3)
    r = O.haar_orthogonal(d, 42)
    eye = torch.eye(d)
    g = torch.Generator().manual_seed(21)
    k = torch.randn(7, d, generator=g) * torch.tensor([0.1, 1, 3, 10, 0.5, 2, 1]).reshape(7, 1)
    idx, norms, signs, gamma = O.prod_quantize(k, r, b3, c3, eye)
    k_mse = O.mse_dequantize(idx, norms, r, c3)
    resid = k - k_mse
    assert torch.equal(signs, torch.where(resid >= 0, 1.0, -1.0))
    q = torch.where(resid >= 0, 1.0, -1.0)
    est = O.prod_inner_product(q, idx, norms, signs, gamma, r, c3, eye).squeeze(-1).double()
    want = (q.double() * k_mse.double()).sum(-1) + resid.double().norm(dim=-1) * math.sqrt(math.pi / 2.0)
    assert torch.allclose(est, want, rtol=2e-5, atol=1e-5)
    for j in (0, 5, 127):
        e = torch.zeros(7, d)
        e[:, j] = 1.0
        est = O.prod_inner_product(e, idx, norms, signs, gamma, r, c3, eye).squeeze(-1).double()
        want = k_mse[:, j].double() + resid.double().norm(dim=-1) * math.sqrt(math.pi / 2.0) / d * q[:, j].double()
        assert torch.allclose(est, want, rtol=2e-5, atol=1e-6)


def test_prod_sketch_term_expectation_over_sketches():
    """E_S[ sqrt(pi/2) / m * <S q, sign(S r)> ] = <q, r> / (|r| sqrt(m)) for S = G / sqrt(m), G
    Gaussian (each row: E[(g.q) sign(g.r)] = sqrt(2/pi) <q, r> / |r|): the correction the
    reference adds is 1 / sqrt(m) of <q, residual>, the consequence of dividing the sketch by
    sqrt(m) and the sum by m (src/flashquant/core/quantizer.py:264-268, 363-368).  Averaged over
    400 sketches the oracle's term must land there within 10 %."""
    d = 64
    c3, b3 = O.lloyd_max_gaussian(d, 3)
    r = O.haar_orthogonal(d, 42)
    g = torch.Generator().manual_seed(3)
    k = torch.randn(1, d, generator=g)
    idx, norms = O.mse_quantize(k, r, b3)
    k_mse = O.mse_dequantize(idx, norms, r, c3)
    resid = k - k_mse
    q = 3.0 * resid / resid.norm() + 0.3 * torch.randn(1, d, generator=g)     # well aligned with the residual
    terms = []
    for seed in range(400):
        s = O.qjl_matrix(d, 1000 + seed)
        _, _, signs, gamma = O.prod_quantize(k, r, b3, c3, s)
        est = O.prod_inner_product(q, idx, norms, signs, gamma, r, c3, s)
        terms.append((est - (q * k_mse).sum(-1, keepdim=True)).item())
    mean = sum(terms) / len(terms)
    want = (q * resid).sum().item() / math.sqrt(d)
    assert want > 0.3
    assert abs(mean - want) < 0.1 * want


def test_prod_estimator_gain_over_many_keys():
    """One sketch, many keys: the sketch term moves the mean error of the MSE-only product by
    1 / sqrt(m) of it, towards zero (the same closed form as above, averaged over keys whose
    residual directions are spread over the sphere)."""
    d = 128
    c3, b3 = O.lloyd_max_gaussian(d, 3)
    r, s = O.haar_orthogonal(d, 42), O.qjl_matrix(d, 42)
    g = torch.Generator().manual_seed(77)
    k = torch.randn(20000, d, generator=g)
    q = k * 0.5 + torch.randn(20000, d, generator=g) * 0.5
    idx, norms, signs, gamma = O.prod_quantize(k, r, b3, c3, s)
    est = O.prod_inner_product(q, idx, norms, signs, gamma, r, c3, s).squeeze(-1)
    true = (q * k).sum(-1)
    mse_only = (q * O.mse_dequantize(idx, norms, r, c3)).sum(-1)
    bias, bias_mse = (est - true).mean().item(), (mse_only - true).mean().item()
    expected_gain = -bias_mse / math.sqrt(d)
    assert expected_gain > 0.1
    assert abs((bias - bias_mse) - expected_gain) < 0.1 * expected_gain + 0.02
    assert abs(bias) < abs(bias_mse)


# ---- TurboQuantProd pages (composition) ---------------------------------------------

def test_prod_page_scores_equal_the_estimator_formula():
    """prod_paged_decode's scores are prod_inner_product's, through the packed page."""
    import math
    d, h, L, bs = 128, 2, 37, 16
    c3, b3 = O.lloyd_max_gaussian(d, 3)
    c4, b4 = O.lloyd_max_gaussian(d, 4)
    r = O.haar_orthogonal(d, 42)
    s = O.qjl_matrix(d, 42)
    g = torch.Generator().manual_seed(5)
    k = torch.randn(L, h, d, generator=g)
    v = torch.randn(L, h, d, generator=g)
    q = torch.randn(1, h, d, generator=g)          # one query head per KV head, float32: no rounding of q_rot
    idx, kn, sg, gam = O.prod_quantize(k, r, b3, c3, s)
    assert int(idx.max()) <= 7 and set(sg.unique().tolist()) <= {-1.0, 1.0}
    kp = O.prod_pack_keys(idx, sg)
    # the nibble carries both fields
    nib = O.nibble_unpack(kp)
    assert torch.equal(nib & 7, idx) and torch.equal(1.0 - 2.0 * (nib >> 3).float(), sg)
    vp, vn = O.compress(v, r, b4)
    nb = (L + bs - 1) // bs
    cache = torch.zeros(nb, bs, O.prod_page_layout(h, d)[4], dtype=torch.uint8)
    table = torch.arange(nb).flip(0).reshape(1, nb).int()
    t = torch.arange(L)
    O.prod_store_rows(cache, table[0].long()[t // bs] * bs + t % bs, kp, kn, gam, vp, vn)
    got = O.prod_paged_decode(q, cache, table, torch.tensor([L], dtype=torch.int32), c3, c4, r, s, h, d, bs)
    # explicit: estimator scores -> softmax -> original-space TQ4 values
    want = torch.zeros(1, h, d)
    for head in range(h):
        sc = O.prod_inner_product(q[0, head].expand(L, d), idx[:, head], kn[:, head], sg[:, head], gam[:, head], r, c3, s)
        w = torch.softmax(sc.reshape(L) / math.sqrt(d), dim=0)
        vv = O.mse_dequantize(O.nibble_unpack(vp[:, head]), vn[:, head], r, c4)
        want[0, head] = w @ vv
    assert (got - want).abs().max().item() < 2e-5
