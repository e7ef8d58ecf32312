"""Fused mode over pre-allocated compressed buffers (the reference's ring buffer,
src/flashquant/cache/buffer_pool.py:21-140, and the fused mode of its HF cache,
src/flashquant/cache/hf_cache.py:322-329, 387-414): keys and values are compressed straight
into (B, H, max_seq, D/2) buffers and the attention kernel reads the valid part through
strided views, without a copy."""
from __future__ import annotations

import pytest
import torch

from oracle import tq_oracle as O
from tests.conftest import outlier_rows
from tests.gpu_util import book

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from flashquant_amd import kernels as K
    from flashquant_amd import load_native
    from flashquant_amd.cache import CompressedBuffer, CompressedKVLayer

DEV = "cuda:0"


@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_strided_views_equal_contiguous_copies_bit_for_bit(d, dtype):
    c, bnd, r = book(d)
    B, H, HQ, cap, n = 2, 2, 8, 300, 171
    g = torch.Generator().manual_seed(5 + d)
    kbuf = torch.randint(0, 256, (B, H, cap, d // 2), dtype=torch.uint8, generator=g).to(DEV)
    vbuf = torch.randint(0, 256, (B, H, cap + 40, d // 2), dtype=torch.uint8, generator=g).to(DEV)   # another capacity
    knb = (torch.rand(B, H, cap, 1, generator=g) * 10 + 0.1).to(DEV)
    vnb = (torch.rand(B, H, cap + 40, 1, generator=g) * 10 + 0.1).to(DEV)
    q = torch.randn(B, HQ, 50, d, generator=g).to(dtype).to(DEV)
    views = (kbuf[:, :, :n], knb[:, :, :n], vbuf[:, :, :n], vnb[:, :, :n])
    assert not views[0].is_contiguous() and not views[2].is_contiguous()
    cd, rd = c.to(DEV), r.to(DEV)
    for causal in (False, True):
        strided = K.fused_tq_attention(q, *views, cd, cd, rd, is_causal=causal)
        copied = K.fused_tq_attention(q, *(t.contiguous() for t in views), cd, cd, rd, is_causal=causal)
        assert torch.equal(strided, copied)
    # single batch and single head: the strides of size-1 dimensions carry no information
    one = K.fused_tq_attention(q[:1, :4], kbuf[:1, :1, :n], knb[:1, :1, :n], vbuf[:1, :1, :n], vnb[:1, :1, :n], cd, cd, rd)
    ref = K.fused_tq_attention(q[:1, :4].contiguous(), kbuf[:1, :1, :n].contiguous(), knb[:1, :1, :n].contiguous(),
                               vbuf[:1, :1, :n].contiguous(), vnb[:1, :1, :n].contiguous(), cd, cd, rd)
    assert torch.equal(one, ref)


@pytest.mark.parametrize("d,dtype", [(128, torch.bfloat16), (128, torch.float16), (64, torch.bfloat16), (256, torch.float16)])
def test_append_in_place_equals_compress_then_append(d, dtype):
    c, bnd, r = book(d)
    B, H, cap = 2, 3, 200
    C = load_native()
    ev, od = C.split_rotation(r)
    ev, od, bd = ev.to(DEV), od.to(DEV), bnd.to(DEV)
    fused = CompressedBuffer(cap, B, H, d // 2, device=torch.device(DEV))
    plain = CompressedBuffer(cap, B, H, d // 2, device=torch.device(DEV))
    for buf in (fused, plain):                     # what lies beyond the valid part must stay untouched
        buf._indices.fill_(0xAB)
        buf._norms.fill_(-7.0)
    for step, n in enumerate([70, 1, 1, 33, 64]):
        x = outlier_rows(B * H * n, 1, d, 300 + step, dtype=dtype).reshape(B, H, n, d).to(DEV)
        fused.append_from(x, ev, od, bd)
        p, nrm = K.tq4_compress(x.reshape(B * H * n, 1, d), r.to(DEV), bd)
        plain.append(p.reshape(B, H, n, d // 2), nrm.reshape(B, H, n, 1))
        assert fused.length == plain.length
    assert torch.equal(fused._indices, plain._indices) and torch.equal(fused._norms, plain._norms)
    assert (fused._indices[:, :, fused.length:] == 0xAB).all() and (fused._norms[:, :, fused.length:] == -7.0).all()
    # and against the oracle on the whole valid part
    idx, nrm = fused.get()
    with pytest.raises(RuntimeError, match="overflow"):
        fused.append_from(torch.zeros(B, H, cap, d, dtype=dtype, device=DEV), ev, od, bd)
    assert idx.shape == (B, H, 169, d // 2) and nrm.shape == (B, H, 169, 1)


def test_append_of_more_than_a_million_tokens_at_once():
    """A long prompt appended in one call: with 2^20 tokens or more per (batch, head) pair the kernel
    finds the pair of a row by comparison instead of by the float32 quotient.  Bit-equal to the plain
    compress of the same rows, in place at the position, everything else untouched."""
    d, dtype = 64, torch.bfloat16
    c, bnd, r = book(d)
    B, H, n = 1, 2, (1 << 20) + 37
    cap = n + 5
    C = load_native()
    ev, od = C.split_rotation(r)
    ev, od, bd = ev.to(DEV), od.to(DEV), bnd.to(DEV)
    buf = CompressedBuffer(cap, B, H, d // 2, device=torch.device(DEV))
    buf._indices.fill_(0xAB)
    buf._norms.fill_(-7.0)
    first = outlier_rows(B * H * 3, 1, d, 400, dtype=dtype).reshape(B, H, 3, d).to(DEV)
    buf.append_from(first, ev, od, bd)
    g = torch.Generator(device=DEV).manual_seed(401)
    x = torch.randn(B, H, n, d, generator=g, device=DEV).to(dtype)
    buf.append_from(x, ev, od, bd)
    p, nrm = K.tq4_compress(x.reshape(B * H * n, 1, d), r.to(DEV), bd)
    assert torch.equal(buf._indices[:, :, 3:3 + n], p.reshape(B, H, n, d // 2))
    assert torch.equal(buf._norms[:, :, 3:3 + n], nrm.reshape(B, H, n, 1))
    assert (buf._indices[:, :, 3 + n:] == 0xAB).all() and (buf._norms[:, :, 3 + n:] == -7.0).all()
    p0, n0 = K.tq4_compress(first.reshape(B * H * 3, 1, d), r.to(DEV), bd)
    assert torch.equal(buf._indices[:, :, :3], p0.reshape(B, H, 3, d // 2))


def test_append_then_attend_matches_the_oracle():
    """A cache step of the fused mode: prefill 150 tokens, then three decode steps of one token
    each, attention over the growing buffers read in place."""
    c, bnd, r = book(128)
    B, HKV, HQ, d, cap = 2, 2, 8, 128, 256
    layer = CompressedKVLayer(cap, B, HKV, d, r, c, bnd, device=torch.device(DEV))
    g = torch.Generator().manual_seed(77)
    ks, vs = [], []
    for n in (150, 1, 1, 1):
        k = torch.randn(B, HKV, n, d, generator=g).to(torch.bfloat16)
        v = torch.randn(B, HKV, n, d, generator=g).to(torch.bfloat16)
        q = torch.randn(B, HQ, n, d, generator=g).to(torch.bfloat16)
        ks.append(k)
        vs.append(v)
        layer.update(k.to(DEV), v.to(DEV))
        got = layer.attend(q.to(DEV), is_causal=n > 1)
        k_all, v_all = torch.cat(ks, 2), torch.cat(vs, 2)
        L = k_all.shape[2]
        kp, kn = O.compress(k_all.reshape(-1, 1, d), r, bnd)
        vp, vn = O.compress(v_all.reshape(-1, 1, d), r, bnd)
        want = O.fused_tq_attention(q, kp.reshape(B, HKV, L, d // 2), kn.reshape(B, HKV, L, 1),
                                    vp.reshape(B, HKV, L, d // 2), vn.reshape(B, HKV, L, 1), c, c, r, is_causal=n > 1)
        assert layer.length == L
        # the kernel's own index choices may differ from the oracle's on at most 1e-4 of the
        # entries; the attention result is compared at the usual bar
        assert (got.cpu().float() - want.float()).abs().max().item() <= 2e-2
