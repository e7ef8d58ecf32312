"""GPU parity at the sizes the benchmark times, and on the magnitudes the reference's
adversarial tests use (tests/test_adversarial.py:13-152: constant rows of 1e6, one
coordinate of 1e8 among 1e-8, rows of 1e-30, zero rows), pushed through decode and prefill.

The oracle is the checker.  At full size it is run on the whole problem where that takes
seconds (paged decode) and on slices where it does not (8192-token prefill: a causal row i
is the non-causal attention of that row over keys 0..i)."""
from __future__ import annotations

import math

import pytest
import torch

from oracle import tq_oracle as O
from tests.conftest import outlier_rows
from tests.gpu_util import book

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from flashquant_amd import kernels as K

DEV = "cuda:0"


def _store_sequences(lens, kv_rows, hkv, d, bs, seed, extra_blocks=0):
    """Paged TQ4 cache holding kv_rows(s, L) -> (k, v) float32 (L, hkv, d) for every sequence,
    compressed by the oracle, behind a seeded random block table."""
    c, b, r = book(d)
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    max_blocks = max(1, (max(lens) + bs - 1) // bs)
    nb = S * max_blocks + extra_blocks
    cache = torch.zeros(nb, bs, hkv * (d + 8), dtype=torch.uint8)
    table = torch.randperm(nb, generator=g)[: S * max_blocks].reshape(S, max_blocks).int()
    for s, L in enumerate(lens):
        if L == 0:
            continue
        k, v = kv_rows(s, L)
        kp, kn = O.compress(k, r, b)
        vp, vn = O.compress(v, r, b)
        t = torch.arange(L)
        O.store_rows(cache, table[s].long()[t // bs] * bs + t % bs, kp, kn, vp, vn)
    return cache, table, torch.tensor(lens, dtype=torch.int32)


def _scaled_tol(want):
    return 2e-2 * max(1.0, want.float().abs().max().item())


# ---- the benchmark's decode workload, exactly ---------------------------------------------------

def test_paged_decode_at_the_benchmark_size():
    """Batch 32, 4096 tokens of context each, 32 query heads over 8 KV heads, 16-token pages,
    N(0,1) rows with four x10 outlier channels per head, block table a seeded permutation."""
    c, b, r = book(128)
    B, L, hq, hkv, bs = 32, 4096, 32, 8, 16

    def rows(s, n):
        return outlier_rows(n, hkv, 128, 5000 + 2 * s), outlier_rows(n, hkv, 128, 5001 + 2 * s)

    cache, table, sl = _store_sequences([L] * B, rows, hkv, 128, bs, seed=2002, extra_blocks=3)
    q = torch.randn(B, hq, 128, generator=torch.Generator().manual_seed(1002)).to(torch.bfloat16)
    want = O.split_k_paged_decode(q, cache, table, sl, c, c, r, hkv, 128, bs)
    cd = c.to(DEV)
    got = K.split_k_paged_decode(q.to(DEV), cache.to(DEV), table.to(DEV), sl.to(DEV), cd, cd, r.to(DEV), hkv, 128, bs)
    # the outlier channels make some output rows reach |x| > 4, where one bfloat16 step is 0.03:
    # 2e-2 of the row's magnitude (never less than 2e-2 absolute)
    assert torch.isfinite(got).all()
    row_scale = want.float().abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
    rel = ((got.cpu().float() - want.float()).abs() / row_scale).max().item()
    assert rel <= 2e-2, f"max error {rel} of the row magnitude"


@pytest.mark.parametrize("hq,hkv,bs", [(16, 4, 16), (16, 2, 32), (8, 1, 16)])
def test_paged_decode_of_few_kv_heads_on_long_ragged_contexts(hq, hkv, bs):
    """4, 2 and 1 KV heads (rows of 2, 4 and 8 tokens in the staged kernel) at contexts of thousands of tokens,
    lengths that leave every kind of last row, the library's own split count: against the oracle, and the direct
    kernel agrees."""
    c, b, r = book(128)
    lens = [4096, 4095, 2049, 1, 3001, 0, 4033, 640, 8193, 5003]

    def rows(s, n):
        return outlier_rows(n, hkv, 128, 6000 + 2 * s), outlier_rows(n, hkv, 128, 6001 + 2 * s)

    cache, table, sl = _store_sequences(lens, rows, hkv, 128, bs, seed=2102, extra_blocks=5)
    q = torch.randn(len(lens), hq, 128, generator=torch.Generator().manual_seed(1102)).to(torch.bfloat16)
    want = O.split_k_paged_decode(q, cache, table, sl, c, c, r, hkv, 128, bs)
    cd = c.to(DEV)
    args = (q.to(DEV), cache.to(DEV), table.to(DEV), sl.to(DEV), cd, cd, r.to(DEV), hkv, 128, bs)
    got = K.split_k_paged_decode(*args)
    from flashquant_amd import load_native
    C = load_native()
    old = C.set_option("decode_direct", True)
    try:
        direct = K.split_k_paged_decode(*args)
    finally:
        C.set_option("decode_direct", old)
    assert torch.isfinite(got).all()
    row_scale = want.float().abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
    for out in (got, direct):
        rel = ((out.cpu().float() - want.float()).abs() / row_scale).max().item()
        assert rel <= 2e-2, f"max error {rel} of the row magnitude"
    assert (got[5] == 0).all()          # the empty sequence


# ---- the benchmark's prefill workload on slices -------------------------------------------------

def test_fused_prefill_at_the_benchmark_size():
    """Batch 4, 8192 tokens, 32 query heads over 8 KV heads, causal.  The GPU computes the whole
    problem; the oracle checks (batch, head, row) samples, among them the first and last rows,
    both sides of a 64-token tile edge and of the workgroup edges."""
    c, bnd, r = book(128)
    B, hq, hkv, N, d = 4, 32, 8, 8192, 128
    g = torch.Generator().manual_seed(1003)
    q = torch.randn(B, hq, N, d, generator=g).to(torch.bfloat16)
    k = outlier_rows(B * hkv * N, 1, d, 6001).reshape(B, hkv, N, d)
    v = outlier_rows(B * hkv * N, 1, d, 6002).reshape(B, hkv, N, d)
    kp, kn = O.compress(k.reshape(-1, 1, d), r, bnd)
    vp, vn = O.compress(v.reshape(-1, 1, d), r, bnd)
    del k, v
    kp, vp = kp.reshape(B, hkv, N, d // 2), vp.reshape(B, hkv, N, d // 2)
    kn, vn = kn.reshape(B, hkv, N, 1), vn.reshape(B, hkv, N, 1)
    got = K.fused_tq_attention(q.to(DEV), kp.to(DEV), kn.to(DEV), vp.to(DEV), vn.to(DEV), c.to(DEV), c.to(DEV),
                               r.to(DEV), is_causal=True)
    torch.cuda.synchronize()
    got = got.cpu().float()
    assert torch.isfinite(got).all()
    rows = [0, 1, 31, 32, 63, 64, 65, 127, 128, 1000, 4095, 4096, 6000, 8127, 8128, 8190, 8191]
    pairs = [(0, 0), (1, 13), (2, 21), (3, 31), (0, 7), (3, 16)]
    worst = 0.0
    for bi, h in pairs:
        hk = h // (hq // hkv)
        for i in rows:
            want = O.fused_tq_attention(q[bi:bi + 1, h:h + 1, i:i + 1], kp[bi:bi + 1, hk:hk + 1, :i + 1],
                                        kn[bi:bi + 1, hk:hk + 1, :i + 1], vp[bi:bi + 1, hk:hk + 1, :i + 1],
                                        vn[bi:bi + 1, hk:hk + 1, :i + 1], c, c, r, is_causal=False)
            err = (got[bi, h, i] - want[0, 0, 0].float()).abs().max().item()
            worst = max(worst, err)
            assert err <= _scaled_tol(want), f"batch {bi} head {h} row {i}: max abs error {err}"
    # a full (batch, head) pair at a quarter of the length would not see the long rows; the last
    # 64 rows of one pair are compared in full instead
    bi, h = 2, 5
    hk = h // (hq // hkv)
    kd = O.decompress(kp[bi, hk].reshape(-1, 1, d // 2), kn[bi, hk].reshape(-1, 1, 1), c).reshape(N, d)
    vd = O.decompress(vp[bi, hk].reshape(-1, 1, d // 2), vn[bi, hk].reshape(-1, 1, 1), c).reshape(N, d)
    q_rot = torch.matmul(q[bi, h, -64:].float(), r.T).to(torch.bfloat16).float()
    sc = (q_rot @ kd.T) / math.sqrt(d)
    sc = sc.masked_fill(torch.arange(N)[None, :] > (N - 64 + torch.arange(64))[:, None], float("-inf"))
    want = torch.matmul(torch.softmax(sc, -1) @ vd, r).to(torch.bfloat16).float()
    sdpa = torch.nn.functional.scaled_dot_product_attention(
        q_rot[None], kd[None], vd[None], attn_mask=(sc > float("-inf"))[None])[0]
    assert (sdpa @ r - want).abs().max() < 2e-2          # the hand-written mask against the library routine
    assert (got[bi, h, -64:] - want).abs().max().item() <= _scaled_tol(want)


# ---- long TurboQuantProd contexts ----------------------------------------------------------------

def test_prod_paged_decode_on_long_ragged_contexts():
    """Three sequences of the long-context workload's shape (64 query heads over 8 KV heads):
    16K, 70K and 128K tokens, the lengths at which the page ids of a split no longer fit one
    register and the chunks are sized inside the kernel."""
    c3, b3 = O.lloyd_max_gaussian(128, 3)
    c4, b4 = O.lloyd_max_gaussian(128, 4)
    r, s = O.haar_orthogonal(128, 42), O.qjl_matrix(128, 42)
    hq, hkv, d, bs = 64, 8, 128, 16
    lens = [16384, 70001, 131072]
    g = torch.Generator().manual_seed(1004)
    max_blocks = (max(lens) + bs - 1) // bs
    nb = sum((L + bs - 1) // bs for L in lens) + 5
    row_bytes = O.prod_page_layout(hkv, d)[4]
    cache = torch.zeros(nb, bs, row_bytes, dtype=torch.uint8)
    perm = torch.randperm(nb, generator=g)
    table = torch.zeros(len(lens), max_blocks, dtype=torch.int32)
    used = 0
    for i, L in enumerate(lens):
        n_pages = (L + bs - 1) // bs
        table[i, :n_pages] = perm[used:used + n_pages].int()
        used += n_pages
        for t0 in range(0, L, 32768):                       # bounded memory on the CPU side
            n = min(32768, L - t0)
            kk = torch.randn(n, hkv, d, generator=g)
            vv = torch.randn(n, hkv, d, generator=g)
            idx, kn, sg, gam = O.prod_quantize(kk, r, b3, c3, s)
            vp, vn = O.compress(vv, r, b4)
            t = torch.arange(t0, t0 + n)
            O.prod_store_rows(cache, table[i].long()[t // bs] * bs + t % bs, O.prod_pack_keys(idx, sg), kn, gam, vp, vn)
    q = torch.randn(len(lens), hq, d, generator=g).to(torch.bfloat16)
    sl = torch.tensor(lens, dtype=torch.int32)
    want = O.prod_paged_decode(q, cache, table, sl, c3, c4, r, s, hkv, d, bs)
    got = K.prod_paged_decode(q.to(DEV), cache.to(DEV), table.to(DEV), sl.to(DEV), c3.to(DEV), c4.to(DEV), r.to(DEV),
                              s.to(DEV), hkv, d, bs)
    torch.cuda.synchronize()
    err = (got.cpu().float() - want.float()).abs().max().item()
    assert math.isfinite(err) and err <= 2e-2, f"max abs error {err}"


@pytest.mark.parametrize("hq,hkv,L", [(32, 8, 4096), (8, 1, 4093), (8, 2, 4090)])
def test_serving_step_at_the_benchmark_size(hq, hkv, L):
    """The benchmark's serving step: batch 32, 4096 tokens of context of which the last is the step's new token,
    stored and attended over in one call (fq_tq4_store_and_decode); and the shards of that model over 8 and 4
    GPUs (1 and 2 KV heads, the new token in the middle of a row of the kernel).  The oracle stores its own
    compress of the same rows and decodes; every sequence is compared."""
    c, b, r = book(128)
    B, bs = 32, 16

    def rows(s, n):
        return outlier_rows(n, hkv, 128, 6000 + 2 * s), outlier_rows(n, hkv, 128, 6001 + 2 * s)

    # the cache holds tokens 0 .. L - 2; position L - 1 holds the bytes of an older token until the step writes it
    cache, table, _ = _store_sequences([L] * B, rows, hkv, 128, bs, seed=2003, extra_blocks=3)
    slots = (table.long()[:, (L - 1) // bs] * bs + (L - 1) % bs).contiguous()
    key = outlier_rows(B, hkv, 128, 7001).to(torch.bfloat16)
    value = outlier_rows(B, hkv, 128, 7002).to(torch.bfloat16)
    q = torch.randn(B, hq, 128, generator=torch.Generator().manual_seed(1003)).to(torch.bfloat16)
    sl = torch.full((B,), L, dtype=torch.int32)
    ref_cache = cache.clone()
    kp, kn = O.compress(key.float(), r, b)
    vp, vn = O.compress(value.float(), r, b)
    O.store_rows(ref_cache, slots, kp, kn, vp, vn)
    want = O.split_k_paged_decode(q, ref_cache, table, sl, c, c, r, hkv, 128, bs)
    cache_d, cd = cache.to(DEV), c.to(DEV)
    got = K.tq4_store_and_decode(key.to(DEV), value.to(DEV), slots.to(DEV), q.to(DEV), cache_d, table.to(DEV), sl.to(DEV),
                                 cd, cd, r.to(DEV), b.to(DEV), hkv, 128, bs)
    torch.cuda.synchronize()
    assert torch.isfinite(got).all()
    row_scale = want.float().abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
    rel = ((got.cpu().float() - want.float()).abs() / row_scale).max().item()
    assert rel <= 2e-2, f"max error {rel} of the row magnitude"
    # the stored rows against the oracle's: an index differs by one bucket at most, and only where the coordinate
    # (rotated in float64) lies within float32 rounding of a bucket boundary; the rest of the cache untouched
    flat_got, flat_ref = cache_d.cpu().reshape(-1, hkv * 136), ref_cache.reshape(-1, hkv * 136)
    keep = torch.ones(flat_got.shape[0], dtype=torch.bool)
    keep[slots] = False
    assert torch.equal(flat_got[keep], flat_ref[keep])
    half = hkv * 68
    for base, rows_in in ((0, key), (half, value)):
        i1 = O.nibble_unpack(flat_got[slots][:, base:base + hkv * 64].contiguous())
        i2 = O.nibble_unpack(flat_ref[slots][:, base:base + hkv * 64].contiguous())
        assert (i1.int() - i2.int()).abs().max().item() <= 1
        for row, col in (i1 != i2).nonzero().tolist():
            x = rows_in[row].reshape(hkv, 128)[col // 128].double()
            y = (r.double() @ (x / (x.norm() + 1e-10)))[col % 128]
            assert (b.double() - y).abs().min().item() <= 1e-6, (row, col)


def test_prod_paged_decode_at_the_benchmark_batch():
    """The long-context workload at its real batch: 8 sequences, lengths drawn uniformly from 16K to
    128K tokens with seed 1004, 64 query heads over 8 KV heads, N(0,1) rows with outlier channels.
    The pages are written by the library's own TurboQuantProd compress (covered against the oracle
    elsewhere); the decode of every sequence runs in one call, and three of the eight (the shortest,
    the longest and one in between) are checked against the oracle on the same pages."""
    from tests.conftest import outlier_rows as rows_cpu
    c3, b3 = O.lloyd_max_gaussian(128, 3)
    c4, b4 = O.lloyd_max_gaussian(128, 4)
    r, s = O.haar_orthogonal(128, 42), O.qjl_matrix(128, 42)
    hq, hkv, d, bs, nseq = 64, 8, 128, 16, 8
    g = torch.Generator(device="cpu").manual_seed(1004)
    lens = torch.randint(16384, 131072 + 1, (nseq,), generator=g)
    pages = (lens + bs - 1) // bs
    total_pages, max_pages = int(pages.sum()), int(pages.max())
    row_bytes = K.prod_page_layout(hkv, d)[4]
    cache = torch.zeros(total_pages, bs, row_bytes, dtype=torch.uint8, device=DEV)
    perm = torch.randperm(total_pages, generator=g)
    table = torch.zeros(nseq, max_pages, dtype=torch.int32)
    rd, sd, b3d, c3d, b4d = r.to(DEV), s.to(DEV), b3.to(DEV), c3.to(DEV), b4.to(DEV)
    first = 0
    for i in range(nseq):
        L, npg = int(lens[i]), int(pages[i])
        table[i, :npg] = perm[first:first + npg].int()
        first += npg
        t = torch.arange(L)
        slots = (table[i].long()[t // bs] * bs + t % bs).to(DEV)
        for t0 in range(0, L, 32768):                       # bounded memory
            n = min(32768, L - t0)
            kx = rows_cpu(n, hkv, d, 1400 + 16 * i + t0 // 32768).to(torch.bfloat16).to(DEV)
            vx = rows_cpu(n, hkv, d, 1500 + 16 * i + t0 // 32768).to(torch.bfloat16).to(DEV)
            kp, kn, kg = K.prod_compress(kx, rd, sd, b3d, c3d)
            vp, vn = K.tq4_compress(vx, rd, b4d)
            K.prod_store_rows(cache, slots[t0:t0 + n], kp, kn, kg, vp, vn)
    q = torch.randn(nseq, hq, d, generator=g).to(torch.bfloat16)
    sl = lens.to(torch.int32)
    got = K.prod_paged_decode(q.to(DEV), cache, table.to(DEV), sl.to(DEV), c3d, c4.to(DEV), rd, sd, hkv, d, bs)
    torch.cuda.synchronize()
    got = got.cpu().float()
    assert torch.isfinite(got).all()
    cache_h = cache.cpu()
    order = torch.argsort(lens)
    for i in (int(order[0]), int(order[nseq // 2]), int(order[-1])):
        want = O.prod_paged_decode(q[i:i + 1], cache_h, table[i:i + 1], sl[i:i + 1], c3, c4, r, s, hkv, d, bs)
        # outlier channels push some output rows past |x| = 4, where one bfloat16 step is 0.03: 2e-2 of
        # the row's magnitude (never less than 2e-2 absolute), as for the TQ4 decode above
        row_scale = want[0].float().abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
        rel = ((got[i] - want[0].float()).abs() / row_scale).max().item()
        assert rel <= 2e-2, f"sequence {i} of {int(lens[i])} tokens: max error {rel} of the row magnitude"


def test_compress_at_the_benchmark_size():
    """The standalone compress workload at full size: 32 layers x 65,536 tokens x 8 KV heads = 16,777,216
    bfloat16 rows of 128 coordinates (N(0,1) with four x10 outlier channels per head), one call.
    Properties over every row, computed on the GPU with torch: the stored norms equal torch's norms of
    the rows, the rows come back from decompress + rotation with the relative squared error of a
    16-level Lloyd-Max quantiser (0.0095) and no row is off by more than what a 4-bit code allows.
    Against the oracle on a sample of 1,048,576 rows spread over the input: index mismatches on at most
    1e-4 of the entries, packing bit-exact given the indices, norms to 1e-6."""
    c, b, r = book(128)
    hkv, d = 8, 128
    n_tok = 32 * 65536
    x = torch.empty(n_tok, hkv, d, dtype=torch.bfloat16, device=DEV)
    chunk = 262144
    gd = torch.Generator(device=DEV).manual_seed(1001)
    gc = torch.Generator().manual_seed(1001)
    chans = [torch.randperm(d, generator=gc)[:4].to(DEV) for _ in range(hkv)]
    for t0 in range(0, n_tok, chunk):
        xf = torch.randn(chunk, hkv, d, generator=gd, device=DEV)
        for h in range(hkv):
            xf[:, h, chans[h]] *= 10.0
        x[t0:t0 + chunk] = xf.to(torch.bfloat16)
    rd, bd, cd = r.to(DEV), b.to(DEV), c.to(DEV)
    packed, norms = K.tq4_compress(x, rd, bd)
    torch.cuda.synchronize()
    assert packed.shape == (n_tok, hkv, d // 2) and norms.shape == (n_tok, hkv, 1)
    worst_norm, err_sq, ref_sq, worst_row = 0.0, 0.0, 0.0, 0.0
    for t0 in range(0, n_tok, chunk):
        xs = x[t0:t0 + chunk].float()
        want_n = xs.norm(dim=-1, keepdim=True)
        got_n = norms[t0:t0 + chunk]
        worst_norm = max(worst_norm, ((got_n - want_n).abs() / want_n.clamp_min(1e-30)).max().item())
        back = K.tq4_decompress_rotated(packed[t0:t0 + chunk], got_n, cd, rd, torch.bfloat16).float()
        e = ((back - xs) ** 2).sum(dim=-1)
        err_sq += e.sum().item()
        ref_sq += (xs ** 2).sum().item()
        worst_row = max(worst_row, (e / (xs ** 2).sum(dim=-1).clamp_min(1e-30)).max().item())
    assert worst_norm <= 1e-5, worst_norm
    rel = err_sq / ref_sq
    assert 0.0085 <= rel <= 0.0105, rel
    assert worst_row <= 0.1, worst_row
    # the oracle on 16 slices of 8192 tokens (x 8 heads = 1,048,576 rows)
    mismatched, entries = 0, 0
    for k in range(16):
        t0 = k * (n_tok // 16) + 4099 * k
        xs = x[t0:t0 + 8192].cpu()
        idx_want, norms_want, _ = O.compress_indices(xs, r, b)
        got_p = packed[t0:t0 + 8192].cpu()
        idx_got = O.nibble_unpack(got_p)
        mismatched += int((idx_got != idx_want).sum().item())
        entries += idx_want.numel()
        assert torch.equal(O.nibble_pack(idx_got), got_p)
        assert ((norms[t0:t0 + 8192].cpu() - norms_want).abs() / norms_want.clamp_min(1e-30)).max().item() <= 1e-6
    assert entries == 1048576 * d
    assert mismatched / entries <= 1e-4, mismatched / entries


# ---- magnitudes of the reference's adversarial tests, through decode and prefill ------------------

def _adversarial_rows(kind, n, h, d, seed):
    g = torch.Generator().manual_seed(seed)
    if kind == "ones_1e6":                       # tests/test_adversarial.py:16-34
        return torch.ones(n, h, d) * 1e6
    if kind == "outlier_1e8":                    # :57-78
        x = torch.full((n, h, d), 1e-8)
        x[..., 0] = 1e8
        return x
    if kind == "tiny_1e-30":                     # :140-152
        return torch.randn(n, h, d, generator=g) * 1e-30
    if kind == "zeros":                          # :81-96
        return torch.zeros(n, h, d)
    if kind == "values_1e4":                     # value norms beyond what fp16(norm * centroid) holds
        return torch.randn(n, h, d, generator=g) * (1e4 if seed % 2 else 1.0)   # odd seeds: the value rows
    raise ValueError(kind)


def _biased_queries(shape, seed):
    """N(0,1) + 0.5: every query has a clearly positive product with the all-ones direction, so a
    key of +-1e6 * ones takes all the weight or none whatever the rounding of its 1e7-fold
    amplified score is (a huge key nearly orthogonal to a query would make the comparison a coin
    toss: the kernels hold the centroids in fp16)."""
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) + 0.5).to(torch.bfloat16)


def _mixed_kv(n, h, d, seed, huge_sign=1.0):
    """Ordinary rows, one key with a huge norm along the all-ones direction (it takes all the
    weight or none, see _biased_queries) and value rows spread over 20 binary orders."""
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(n, h, d, generator=g)
    v = torch.randn(n, h, d, generator=g)
    k[n // 3] = huge_sign * 1e6
    scale = torch.ones(n)
    scale[::7] = 3e3
    scale[5::11] = 1e6
    v *= scale[:, None, None]
    return k, v


KINDS = ["ones_1e6", "outlier_1e8", "tiny_1e-30", "zeros", "values_1e4", "mixed"]


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 128), (8, 2, 64)])
def test_paged_decode_on_adversarial_magnitudes(kind, hq, hkv, d):
    c, b, r = book(d)
    lens = [150, 33, 700]

    def rows(s, n):
        if kind == "mixed":
            return _mixed_kv(n, hkv, d, 7000 + s, huge_sign=-1.0 if s == 1 else 1.0)
        return _adversarial_rows(kind, n, hkv, d, 7000 + 2 * s), _adversarial_rows(kind, n, hkv, d, 7101 + 2 * s)

    cache, table, sl = _store_sequences(lens, rows, hkv, d, 16, seed=71, extra_blocks=2)
    q = _biased_queries((len(lens), hq, d), 72)
    want = O.split_k_paged_decode(q, cache, table, sl, c, c, r, hkv, d, 16)
    cd = c.to(DEV)
    for splits in (1, 3):
        got = K.split_k_paged_decode(q.to(DEV), cache.to(DEV), table.to(DEV), sl.to(DEV), cd, cd, r.to(DEV), hkv, d, 16,
                                     num_splits=splits)
        assert torch.isfinite(got).all() and torch.isfinite(want.float()).all()
        # a row's tolerance follows that row's magnitude (value rows span 20 binary orders)
        row_scale = want.float().abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
        rel = ((got.cpu().float() - want.float()).abs() / row_scale).max().item()
        assert rel <= 2e-2, f"{kind} splits={splits}: max error {rel} of the row magnitude"


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (4, 2, 64)])
def test_fused_attention_on_adversarial_magnitudes(kind, hq, hkv, d):
    c, bnd, r = book(d)
    B, N = 2, 200
    if kind == "mixed":
        _, v = _mixed_kv(B * hkv * N, 1, d, 7300)
        k = torch.randn(B * hkv * N, 1, d, generator=torch.Generator().manual_seed(7301))
        for bi in range(B * hkv):                 # one huge key per (batch, head): it wins in batch 0, loses in batch 1
            k[bi * N + 40 + bi] = 1e6 if bi < hkv else -1e6
    else:
        k = _adversarial_rows(kind, B * hkv * N, 1, d, 7200)
        v = _adversarial_rows(kind, B * hkv * N, 1, d, 7201)
    kp, kn = O.compress(k, r, bnd)
    vp, vn = O.compress(v, r, bnd)
    shape_p, shape_n = (B, hkv, N, d // 2), (B, hkv, N, 1)
    kp, kn, vp, vn = kp.reshape(shape_p), kn.reshape(shape_n), vp.reshape(shape_p), vn.reshape(shape_n)
    q = _biased_queries((B, hq, N, d), 73)
    for causal in (True, False):
        want = O.fused_tq_attention(q, kp, kn, vp, vn, c, c, r, is_causal=causal)
        got = K.fused_tq_attention(q.to(DEV), kp.to(DEV), kn.to(DEV), vp.to(DEV), vn.to(DEV), c.to(DEV), c.to(DEV),
                                   r.to(DEV), is_causal=causal)
        torch.cuda.synchronize()
        assert torch.isfinite(got).all() and torch.isfinite(want.float()).all()
        # a row's tolerance follows that row's magnitude: rows before the huge value rows stay small
        row_scale = want.float().abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
        rel = ((got.cpu().float() - want.float()).abs() / row_scale).max().item()
        assert rel <= 2e-2, f"{kind} causal={causal}: max error {rel} of the row magnitude"


@pytest.mark.parametrize("kind", ["ones_1e6", "values_1e4", "mixed"])
def test_paged_prefill_on_adversarial_magnitudes(kind):
    c, b, r = book(128)
    hq, hkv, d = 8, 2, 128
    kv_lens, q_lens = [150, 260], [150, 31]

    def rows(s, n):
        if kind == "mixed":
            return _mixed_kv(n, hkv, d, 7400 + s, huge_sign=-1.0 if s == 1 else 1.0)
        return _adversarial_rows(kind, n, hkv, d, 7400 + 2 * s), _adversarial_rows(kind, n, hkv, d, 7501 + 2 * s)

    cache, table, sl = _store_sequences(kv_lens, rows, hkv, d, 16, seed=74, extra_blocks=2)
    q = _biased_queries((sum(q_lens), hq, d), 75)
    cu = torch.tensor([0, q_lens[0], sum(q_lens)], dtype=torch.int32)
    want = O.paged_prefill(q, cu, cache, table, sl, c, c, r, hkv, d, 16)
    got = K.paged_tq4_prefill(q.to(DEV), cu.to(DEV), max(q_lens), cache.to(DEV), table.to(DEV), sl.to(DEV), c.to(DEV),
                              c.to(DEV), r.to(DEV), hkv, d, 16)
    torch.cuda.synchronize()
    assert torch.isfinite(got).all() and torch.isfinite(want.float()).all()
    row_scale = want.float().abs().amax(dim=-1, keepdim=True).clamp_min(1.0)
    rel = ((got.cpu().float() - want.float()).abs() / row_scale).max().item()
    assert rel <= 2e-2, f"{kind}: max error {rel} of the row magnitude"
