"""GPU checks of the class surface of the reference's C++ bindings (_C.quantizer, csrc/bindings/
quantizer_bind.cpp:10-64) and of the kernel calls of its vLLM attention implementation
(flashquant_amd.vllm.TQ4AttentionKernels, src/flashquant/vllm/impl.py:220-394, 470-512)."""
from __future__ import annotations

import math

import pytest
import torch

from oracle import tq_oracle as O
from tests.conftest import outlier_rows
from tests.gpu_util import book

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from flashquant_amd import load_native
    from flashquant_amd.vllm import TQ4AttentionKernels

DEV = "cuda:0"


@pytest.mark.parametrize("dim,bits", [(128, 4), (64, 3), (256, 2)])
def test_c_quantizer_mse_class(dim, bits):
    C = load_native()
    qz = C.quantizer.TurboQuantMSE(dim, bits, 42)
    c, b = O.lloyd_max_gaussian(dim, bits)
    r = O.haar_orthogonal(dim, 42)
    x = outlier_rows(41, 3, dim, 400 + dim)
    res = qz.quantize(x.to(DEV))
    wi, wn = O.mse_quantize(x, r, b)
    assert res.indices.dtype == torch.int64 and res.indices.shape == x.shape and res.norms.shape == (41, 3, 1)
    assert (res.indices.cpu() != wi).float().mean().item() <= 1e-4
    assert torch.allclose(res.norms.cpu(), wn, rtol=1e-6, atol=0)
    rec = qz.dequantize(res.indices, res.norms)
    want = O.mse_dequantize(res.indices.cpu(), res.norms.cpu(), r, c)
    assert (rec.cpu() - want).abs().max().item() <= 1e-5 * want.abs().max().item()


def test_c_quantizer_prod_class():
    C = load_native()
    dim = 128
    qz = C.quantizer.TurboQuantProd(dim, 4, 42)
    c, b = O.lloyd_max_gaussian(dim, 3)
    r, s = O.haar_orthogonal(dim, 42), O.qjl_matrix(dim, 42)
    x = outlier_rows(50, 3, dim, 500)
    res = qz.quantize(x.to(DEV))
    wi, wn, ws, wg = O.prod_quantize(x, r, b, c, s)
    assert res.qjl_signs.dtype == torch.int8 and res.qjl_signs.shape == x.shape     # int8, as the reference's C++ stores them
    assert set(res.qjl_signs.unique().tolist()) <= {-1, 1}
    assert (res.indices.cpu() != wi).float().mean().item() <= 1e-4
    same = (res.indices.cpu() == wi).all(dim=-1)
    assert (res.qjl_signs.cpu().float()[same] != ws[same]).float().mean().item() <= 1e-3
    assert torch.allclose(res.residual_norms.cpu()[same], wg[same], rtol=1e-4)
    q = torch.randn(50, 3, dim, generator=torch.Generator().manual_seed(6))
    est = qz.estimate_inner_product(q.to(DEV), res).cpu()
    want = O.prod_inner_product(q, res.indices.cpu(), res.norms.cpu(), res.qjl_signs.cpu().float(),
                                res.residual_norms.cpu(), r, c, s)
    assert est.shape == (50, 3, 1)
    assert (est - want).abs().max().item() <= 1e-4 * max(1.0, want.abs().max().item())
    assert torch.equal(qz.dequantize(res.indices, res.norms),
                       C.mse_dequantize(res.indices, res.norms, r.to(DEV), c.to(DEV)))


def test_vllm_shaped_kernel_calls_store_decode_prefill_decompress():
    """A serving step with the four calls the reference's forward() is made of: store the prompt's
    keys and values, prefill over the packed cache, store one more token, decode; then
    materialise the cache as the non-fused path does."""
    c, bnd, r = book(128)
    hq, hkv, d, bs = 32, 8, 128, 16
    ker = TQ4AttentionKernels(hkv, d, 1.0 / math.sqrt(d), torch.device(DEV))
    assert torch.equal(ker.rotation.cpu(), r) and torch.equal(ker.centroids.cpu(), c) and ker.total_bytes == 1088
    g = torch.Generator().manual_seed(88)
    lens = [45, 130]
    S = len(lens)
    max_blocks = 10
    nb = S * max_blocks + 2
    table = torch.randperm(nb, generator=g)[: S * max_blocks].reshape(S, max_blocks).int()
    cache = torch.zeros(nb, bs, 1088, dtype=torch.uint8, device=DEV)
    cache_ref = torch.zeros(nb, bs, 1088, dtype=torch.uint8)
    ks = [torch.randn(L + 1, hkv, d, generator=g).to(torch.bfloat16) for L in lens]   # prompt + one decode token
    vs = [torch.randn(L + 1, hkv, d, generator=g).to(torch.bfloat16) for L in lens]

    def slots_of(s, t0, t1):
        t = torch.arange(t0, t1)
        return table[s].long()[t // bs] * bs + t % bs

    # ---- prompt: store, then prefill over the cache -------------------------------------------
    key = torch.cat([ks[s][:L] for s, L in enumerate(lens)])
    value = torch.cat([vs[s][:L] for s, L in enumerate(lens)])
    slots = torch.cat([slots_of(s, 0, L) for s, L in enumerate(lens)])
    ker.compress_and_store(key.to(DEV), value.to(DEV), cache, slots.to(DEV))
    kp, kn = O.compress(key, r, bnd)
    vp, vn = O.compress(value, r, bnd)
    O.store_rows(cache_ref, slots, kp, kn, vp, vn)
    q = torch.randn(sum(lens), hq, d, generator=g).to(torch.bfloat16)
    cu = torch.tensor([0, lens[0], sum(lens)], dtype=torch.int32)
    sl = torch.tensor(lens, dtype=torch.int32)
    got = ker.prefill(q.to(DEV), cu.to(DEV), max(lens), cache, table.to(DEV), sl.to(DEV))
    want = O.paged_prefill(q, cu, cache_ref, table, sl, c, c, r, hkv, d, bs)
    assert (got.cpu().float() - want.float()).abs().max().item() <= 2e-2
    # ---- one decode step ------------------------------------------------------------------------
    key1 = torch.stack([ks[s][L] for s, L in enumerate(lens)])
    value1 = torch.stack([vs[s][L] for s, L in enumerate(lens)])
    slots1 = torch.cat([slots_of(s, L, L + 1) for s, L in enumerate(lens)])
    ker.compress_and_store(key1.to(DEV), value1.to(DEV), cache, slots1.to(DEV))
    kp1, kn1 = O.compress(key1, r, bnd)
    vp1, vn1 = O.compress(value1, r, bnd)
    O.store_rows(cache_ref, slots1, kp1, kn1, vp1, vn1)
    q1 = torch.randn(S, hq, d, generator=g).to(torch.bfloat16)
    sl1 = sl + 1
    out = torch.empty(S, hq, d, dtype=torch.bfloat16, device=DEV)
    got1 = ker.decode(q1.to(DEV), cache, table.to(DEV), sl1.to(DEV), out=out)
    want1 = O.split_k_paged_decode(q1, cache_ref, table, sl1, c, c, r, hkv, d, bs)
    assert got1.data_ptr() == out.data_ptr()
    assert (got1.cpu().float() - want1.float()).abs().max().item() <= 2e-2
    # ---- materialise the cache ------------------------------------------------------------------
    k_rot, v_rot = ker.decompress_cache(cache, torch.bfloat16, apply_rotation=False)
    k_org, v_org = ker.decompress_cache(cache, torch.bfloat16, apply_rotation=True)
    assert k_rot.shape == (nb, bs, hkv, d) and v_org.shape == (nb, bs, hkv, d)
    got_cache = cache.cpu()
    for s, L in enumerate(lens):
        rows = slots_of(s, 0, L + 1)
        kk, vv = O.gather_sequence(got_cache, table[s], L + 1, c, c, hkv, d, bs)      # (H, L + 1, D) float32, rotated
        assert torch.equal(k_rot.reshape(-1, hkv, d)[rows.to(DEV)].cpu(), kk.permute(1, 0, 2).to(torch.bfloat16))
        want_v = torch.matmul(vv.permute(1, 0, 2).to(torch.bfloat16).float(), r)
        diff = (v_org.reshape(-1, hkv, d)[rows.to(DEV)].cpu().float() - want_v).abs().max().item()
        assert diff <= 2 ** -7 * want_v.abs().max().item()
        # and the round trip: the original-space values are the stored tokens up to the 4-bit distortion
        rel = ((v_org.reshape(-1, hkv, d)[rows.to(DEV)].cpu().float() - vs[s].float()) ** 2).sum() / (vs[s].float() ** 2).sum()
        assert 0.007 <= rel.item() <= 0.012
