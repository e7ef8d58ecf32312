"""The decode entry point that allocates nothing (fq_split_k_paged_decode_static): its split
partials live in the library's static device array instead of a caller workspace.  Checked
against the entry point it is a variant of, on two calls in a row, the second on a smaller
problem (the array then still holds the first call's partials)."""
from __future__ import annotations

import math

import pytest
import torch

from tests.gpu_util import book, build_paged_case

pytestmark = pytest.mark.gpu

if torch.cuda.is_available():
    from flashquant_amd import load_native

DEV = "cuda:0"


def _both(lens, hq, hkv, seed, num_splits=0, d=128, bs=16, dtype=torch.bfloat16):
    C = load_native()
    c, b, r = book(d)
    q, cache, table, sl = build_paged_case(lens, hq, hkv, d=d, bs=bs, seed=seed, dtype=dtype)
    dev = [t.to(DEV).contiguous() for t in (q, cache, table, sl, c, r)]
    scale = 1.0 / math.sqrt(d)
    want = C.split_k_paged_decode(dev[0], dev[1], dev[2], dev[3], dev[4], dev[4], dev[5], hkv, d, bs, scale, None,
                                  num_splits)
    out = torch.full_like(dev[0], float("nan"))
    if not _both.warm:
        # the first call on a device asks the runtime for the static array's address and may load kernel
        # code; callers make it before any region that must not allocate, and so does this test
        C.split_k_paged_decode_static(dev[0], dev[1], dev[2], dev[3], dev[4], dev[4], dev[5], hkv, d, bs, scale,
                                      torch.empty_like(out), num_splits)
        _both.warm = True
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]
    got = C.split_k_paged_decode_static(dev[0], dev[1], dev[2], dev[3], dev[4], dev[4], dev[5], hkv, d, bs, scale,
                                        out, num_splits)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before        # nothing came from torch's allocator
    assert torch.cuda.mem_get_info()[0] == free_before    # nor from the runtime's, around torch (hipMalloc)
    assert got.data_ptr() == out.data_ptr()
    return got, want


_both.warm = False


def test_static_scratch_decode_matches_the_workspace_entry_point_twice():
    # first call: 8 sequences up to 3000 tokens, 32 query heads over 8 KV heads (the staged kernel)
    got, want = _both([3000, 0, 37, 1500, 64, 2049, 1, 777], 32, 8, seed=41)
    assert torch.equal(got, want)
    # second call, smaller in every extent: fewer sequences, shorter contexts, fewer splits
    got, want = _both([129, 5], 32, 8, seed=42, num_splits=2)
    assert torch.equal(got, want)
    # and the kernel for the other shapes, with a split count that leaves most splits empty
    got, want = _both([70, 5, 200], 8, 2, seed=43, num_splits=9, d=64, bs=8, dtype=torch.float16)
    assert torch.equal(got, want)


def test_static_scratch_decode_refuses_what_does_not_fit():
    C = load_native()
    c, b, r = book(128)
    S, hq, hkv, bs = 64, 128, 8, 16
    max_blocks = 4096                                   # 64K tokens of context: 64 x 128 rows x 256 splits of partials
    q = torch.zeros(S, hq, 128, dtype=torch.bfloat16, device=DEV)
    cache = torch.zeros(2, bs, hkv * 136, dtype=torch.uint8, device=DEV)
    table = torch.zeros(S, max_blocks, dtype=torch.int32, device=DEV)
    sl = torch.ones(S, dtype=torch.int32, device=DEV)
    need = C.paged_decode_workspace_bytes(S, hq, hkv, 128, bs, max_blocks, 256)
    assert need > C.static_scratch_bytes()
    with pytest.raises(ValueError, match="workspace"):
        C.split_k_paged_decode_static(q, cache, table, sl, c.to(DEV), c.to(DEV), r.to(DEV), hkv, 128, bs, 0.1,
                                      torch.empty_like(q), 256)
