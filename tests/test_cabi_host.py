"""CPU-only checks of the C ABI: the library loads, exports every symbol that
include/fq_hip.h declares, and rejects bad arguments with status codes before
touching the GPU (the reference's launchers abort() in these cases:
csrc/cuda/compress.cu:276-280, csrc/cuda/paged_decode.cu:401-415)."""
from __future__ import annotations

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "flashquant_amd", "libfq_hip.so")
HEADER = os.path.join(ROOT, "include", "fq_hip.h")

FQ_OK, FQ_NULL, FQ_DIM, FQ_BLOCK, FQ_DTYPE, FQ_SHAPE, FQ_ALIGN, FQ_WS, FQ_LAUNCH = range(9)


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        pytest.fail("libfq_hip.so is not built: run `python -m flashquant_amd.build`")
    return ctypes.CDLL(LIB)


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fq_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported(lib):
    names = declared_symbols()
    assert len(names) >= 10
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in fq_hip.h but not exported"


def test_version_and_status_strings(lib):
    assert lib.fq_abi_version() == 1
    lib.fq_status_string.restype = ctypes.c_char_p
    seen = set()
    for code in range(9):
        text = lib.fq_status_string(code).decode()
        assert text and text not in seen
        seen.add(text)
    assert lib.fq_status_string(99).decode() == "unknown status"


def _p(v=0):
    return ctypes.c_void_p(v)


def test_compress_argument_errors(lib):
    f = lib.fq_tq4_compress
    f.argtypes = [ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 5 + [ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    assert f(_p(), 1, _p(), _p(), _p(), _p(), _p(), 0, 128, _p()) == FQ_OK            # M == 0: no-op
    assert f(_p(), 1, _p(), _p(), _p(), _p(), _p(), -1, 128, _p()) == FQ_SHAPE
    assert f(_p(), 1, _p(), _p(), _p(), _p(), _p(), 4, 96, _p()) == FQ_DIM
    assert f(_p(), 2, _p(), _p(), _p(), _p(), _p(), 4, 128, _p()) == FQ_DTYPE         # float32 rows
    assert f(_p(), 1, _p(), _p(), _p(), _p(), _p(), 4, 128, _p()) == FQ_NULL
    assert f(_p(8), 1, _p(16), _p(16), _p(16), _p(16), _p(16), 4, 128, _p()) == FQ_ALIGN


def test_decompress_argument_errors(lib):
    f = lib.fq_tq4_decompress
    f.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    assert f(_p(), _p(), _p(), _p(), 1, 0, 128, _p()) == FQ_OK
    assert f(_p(), _p(), _p(), _p(), 1, 3, 100, _p()) == FQ_DIM
    assert f(_p(), _p(), _p(), _p(), 7, 3, 128, _p()) == FQ_DTYPE
    assert f(_p(), _p(), _p(), _p(), 1, 3, 128, _p()) == FQ_NULL
    assert f(_p(16), _p(16), _p(16), _p(8), 1, 3, 128, _p()) == FQ_ALIGN


def test_decode_argument_errors_and_sizes(lib):
    f = lib.fq_split_k_paged_decode
    f.argtypes = ([ctypes.c_void_p] * 7 + [ctypes.c_int, ctypes.c_void_p] + [ctypes.c_int] * 6 +
                  [ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                   ctypes.c_void_p])

    def call(S=2, HQ=32, HKV=8, D=128, BS=16, MB=4, NB=64, dtype=1, ns=0, ws=0, wsb=0, ptr=0):
        return f(_p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(), 0, _p(ptr), S, HQ, HKV, D, BS, MB, NB,
                 0.088, dtype, ns, _p(ws), wsb, _p())

    assert call(S=0) == FQ_OK
    assert call(D=80) == FQ_DIM
    assert call(BS=12) == FQ_BLOCK
    assert call(dtype=2) == FQ_DTYPE
    assert call(HQ=30) == FQ_SHAPE            # not a multiple of the KV heads
    assert call(HQ=8 * 17) == FQ_SHAPE        # more than 16 query heads per KV head
    assert call(S=-1) == FQ_SHAPE
    assert call() == FQ_NULL
    assert call(ptr=4096) == FQ_WS            # no workspace given
    lib.fq_paged_decode_workspace_bytes.restype = ctypes.c_size_t
    need = lib.fq_paged_decode_workspace_bytes(2, 32, 8, 128, 16, 4, 3)
    rows = 2 * 32
    assert need >= rows * 3 * 128 * 4 + 2 * rows * 3 * 4 + rows * 128 * 2
    assert call(ptr=4096, ws=4096, wsb=need - 1, ns=3) == FQ_WS
    assert call(ptr=4096, ws=4096 + 8, wsb=need, ns=3) == FQ_ALIGN


def test_split_count_rules(lib):
    # a split spans at most 256 pages
    assert lib.fq_paged_decode_min_splits(16, 256) == 1
    assert lib.fq_paged_decode_min_splits(16, 8192) == 32      # 128K tokens of context
    assert lib.fq_paged_decode_min_splits(8, 8192) == 32
    auto = lib.fq_paged_decode_auto_splits(8, 8, 16, 8192)
    assert auto >= 32
    assert lib.fq_paged_decode_auto_splits(1, 1, 16, 1) == 1
    # fewer than 8 KV heads (the direct kernel): chunks of at least 256 tokens
    assert lib.fq_paged_decode_auto_splits(32, 1, 16, 256) <= 16
    assert lib.fq_paged_decode_auto_splits(32, 2, 16, 256) <= 16
    assert lib.fq_paged_decode_auto_splits(4, 4, 16, 2048) >= 32      # long contexts still fill the chip
    # one long sequence: no more splits than the combine step takes in two passes
    assert lib.fq_paged_decode_auto_splits(1, 8, 16, 2048) == 128
    assert lib.fq_paged_decode_auto_splits(1, 8, 16, 16384) == 128    # 256K tokens: the minimum is 64
    f = lib.fq_paged_tq4_decode
    f.argtypes = ([ctypes.c_void_p] * 2 + [ctypes.c_int] + [ctypes.c_void_p] * 8 + [ctypes.c_int] * 6 +
                  [ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])
    args = [_p(4096), _p(), 0] + [_p(4096)] * 8
    assert f(*args, 1, 8, 8, 128, 16, 8192, 9000, 0.1, 1, 4, _p()) == FQ_SHAPE   # fewer splits than the minimum


def test_rotation_fusion_rule(lib):
    assert lib.fq_paged_decode_fuses_rotation(128, 8, 1) == 1
    assert lib.fq_paged_decode_fuses_rotation(128, 8, 0) == 1    # distinct K and V codebooks share the table
    assert lib.fq_paged_decode_fuses_rotation(64, 8, 1) == 0
    assert lib.fq_paged_decode_fuses_rotation(128, 4, 1) == 0


def test_codebook_solver_runs_on_the_host_and_matches_the_committed_levels(lib):
    import json
    f = lib.fq_lloyd_max_gaussian
    f.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_float), ctypes.POINTER(ctypes.c_float)]
    golden = json.load(open(os.path.join(ROOT, "tests", "golden", "codebook_d128.json")))
    for bits in (2, 3, 4):
        c = (ctypes.c_float * (1 << bits))()
        b = (ctypes.c_float * ((1 << bits) - 1))()
        assert f(128, bits, c, b) == FQ_OK
        want = golden[str(bits)]
        assert max(abs(x - y) for x, y in zip(c, want["centroids"])) < 1e-8
        assert max(abs(x - y) for x, y in zip(b, want["boundaries"])) < 1e-8
        assert all(c[i] < c[i + 1] for i in range(len(c) - 1))
    c = (ctypes.c_float * 2)()
    b = (ctypes.c_float * 1)()
    assert f(128, 0, c, b) == FQ_SHAPE and f(0, 2, c, b) == FQ_SHAPE and f(128, 9, c, b) == FQ_SHAPE
    assert f(128, 1, None, b) == FQ_NULL


def test_quantizer_and_packing_argument_errors(lib):
    q = lib.fq_mse_quantize
    q.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                  ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    assert q(_p(), 2, _p(), 0, _p(), 15, _p(), _p(), 0, 128, _p()) == FQ_OK
    assert q(_p(), 2, _p(), 0, _p(), 16, _p(), _p(), 4, 128, _p()) == FQ_SHAPE       # at most 15 boundaries
    assert q(_p(), 2, _p(), 0, _p(), 15, _p(), _p(), 4, 96, _p()) == FQ_DIM
    assert q(_p(), 5, _p(), 0, _p(), 15, _p(), _p(), 4, 128, _p()) == FQ_DTYPE
    assert q(_p(), 2, _p(), 0, _p(), 15, _p(), _p(), 4, 128, _p()) == FQ_NULL
    assert q(_p(16), 2, _p(8), 0, _p(16), 15, _p(16), _p(16), 4, 128, _p()) == FQ_ALIGN
    d = lib.fq_mse_dequantize
    d.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
                  ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    assert d(_p(), _p(), _p(), 0, _p(), 1, _p(), 4, 128, _p()) == FQ_SHAPE            # fewer than 2 levels
    assert d(_p(), _p(), _p(), 0, _p(), 16, _p(), 4, 128, _p()) == FQ_NULL
    pr = lib.fq_project_rows
    pr.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                   ctypes.c_int64, ctypes.c_int, ctypes.c_void_p]
    assert pr(_p(), 2, _p(), 0, 1, _p(), -1, 128, _p()) == FQ_SHAPE
    assert pr(_p(), 2, _p(), 0, 1, _p(), 3, 32, _p()) == FQ_DIM
    p2 = lib.fq_pack_2bit
    p2.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p]
    assert p2(_p(), 8, _p(), 0, _p(), _p()) == FQ_OK
    assert p2(_p(), 2, _p(), 4, _p(), _p()) == FQ_DTYPE                               # 16-bit indices
    assert p2(_p(), 8, _p(), 4, _p(), _p()) == FQ_NULL


def test_paged_prefill_argument_errors(lib):
    f = lib.fq_paged_tq4_prefill
    f.argtypes = ([ctypes.c_void_p] * 8 + [ctypes.c_int, ctypes.c_void_p] + [ctypes.c_int] * 7 +
                  [ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])

    def call(S=2, maxq=64, HQ=32, HKV=8, D=128, BS=16, MB=4, NB=64, dtype=1, ptr=0, out=None):
        o = ptr if out is None else out
        return f(_p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), 0, _p(o), S, maxq, HQ, HKV, D,
                 BS, MB, NB, 0.088, 1, dtype, _p())

    assert call(S=0) == FQ_OK and call(maxq=0) == FQ_OK
    assert call(HQ=30) == FQ_SHAPE
    assert call(D=100) == FQ_DIM and call(D=64) == FQ_NULL          # 64, 128 and 256 are all served
    assert call(BS=12) == FQ_BLOCK
    assert call(dtype=2) == FQ_DTYPE
    assert call(S=-1) == FQ_SHAPE and call(MB=0) == FQ_SHAPE
    assert call() == FQ_NULL
    assert call(ptr=4096 + 8) == FQ_ALIGN


def test_ring_buffer_and_rotated_decompress_argument_errors(lib):
    ap = lib.fq_tq4_compress_append
    ap.argtypes = ([ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 5 + [ctypes.c_int64] * 4 +
                   [ctypes.c_int, ctypes.c_void_p])
    assert ap(_p(), 1, _p(), _p(), _p(), _p(), _p(), 0, 5, 100, 0, 128, _p()) == FQ_OK        # no slabs: no-op
    assert ap(_p(), 1, _p(), _p(), _p(), _p(), _p(), 4, 5, 100, 96, 128, _p()) == FQ_SHAPE    # 96 + 5 > capacity
    assert ap(_p(), 1, _p(), _p(), _p(), _p(), _p(), 4, 5, 100, -1, 128, _p()) == FQ_SHAPE
    assert ap(_p(), 1, _p(), _p(), _p(), _p(), _p(), 4, 5, 100, 10, 100, _p()) == FQ_DIM
    assert ap(_p(), 2, _p(), _p(), _p(), _p(), _p(), 4, 5, 100, 10, 128, _p()) == FQ_DTYPE
    assert ap(_p(), 1, _p(), _p(), _p(), _p(), _p(), 4, 5, 100, 10, 128, _p()) == FQ_NULL
    at = lib.fq_fused_tq_attention_strided
    at.argtypes = ([ctypes.c_void_p] * 8 + [ctypes.c_int, ctypes.c_void_p] + [ctypes.c_int] * 5 + [ctypes.c_int64] * 2 +
                   [ctypes.c_int, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])

    def att(nkv=64, kcap=64, vcap=64, d=128):
        return at(_p(), _p(), _p(), _p(), _p(), _p(), _p(), _p(), 0, _p(), 1, 8, 2, 16, nkv, kcap, vcap, d, 0.1, 1, 1, _p())

    assert att(kcap=63) == FQ_SHAPE and att(vcap=10) == FQ_SHAPE      # a capacity below the length
    assert att(kcap=1000, vcap=2000) == FQ_NULL                       # accepted, then the NULL operands are found
    assert att(d=96) == FQ_DIM
    big = (1 << 24) + 1
    assert att(nkv=big, kcap=big, vcap=big) == FQ_SHAPE                # beyond the 32-bit offsets of a slab
    dr = lib.fq_tq4_decompress_rotated
    dr.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int,
                                           ctypes.c_void_p]
    assert dr(_p(), _p(), _p(), _p(), 0, _p(), 1, 0, 128, _p()) == FQ_OK
    assert dr(_p(), _p(), _p(), _p(), 0, _p(), 2, 4, 128, _p()) == FQ_DTYPE     # float32 output: not offered
    assert dr(_p(), _p(), _p(), _p(), 0, _p(), 1, 4, 100, _p()) == FQ_DIM
    assert dr(_p(), _p(), _p(), _p(), 0, _p(), 1, 4, 128, _p()) == FQ_NULL
    assert dr(_p(16), _p(16), _p(16), _p(16), 0, _p(8), 1, 4, 128, _p()) == FQ_ALIGN


def test_static_scratch_decode_refuses_before_touching_the_gpu(lib):
    lib.fq_static_scratch_bytes.restype = ctypes.c_size_t
    assert lib.fq_static_scratch_bytes() == 16 << 20
    f = lib.fq_split_k_paged_decode_static
    f.argtypes = ([ctypes.c_void_p] * 7 + [ctypes.c_int, ctypes.c_void_p] + [ctypes.c_int] * 6 +
                  [ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])

    def call(S=4, HQ=32, HKV=8, D=128, BS=16, MB=64, splits=0):
        return f(_p(), _p(), _p(), _p(), _p(), _p(), _p(), 0, _p(), S, HQ, HKV, D, BS, MB, 100, 0.1, 1, splits, _p())

    assert call(S=0) == FQ_OK
    assert call(HQ=30) == FQ_SHAPE and call(D=100) == FQ_DIM and call(BS=12) == FQ_BLOCK
    assert call(S=64, HQ=128, MB=4096, splits=256) == FQ_WS          # 1 GiB of partials against 16 MiB


def test_option_switches(lib):
    assert lib.fq_get_option(99) == -1 and lib.fq_set_option(99, 1) == FQ_SHAPE
    for opt in range(6):
        old = lib.fq_get_option(opt)
        assert old in (0, 1)
        assert lib.fq_set_option(opt, 1 - old) == FQ_OK and lib.fq_get_option(opt) == 1 - old
        assert lib.fq_set_option(opt, old) == FQ_OK and lib.fq_get_option(opt) == old
    # rows per workgroup of the combine kernel: a number, not a switch
    assert lib.fq_get_option(6) == 0
    assert lib.fq_set_option(6, 8) == FQ_OK and lib.fq_get_option(6) == 8
    assert lib.fq_set_option(6, 0) == FQ_OK and lib.fq_get_option(6) == 0


def test_shape_limits_of_the_staged_and_prod_decodes(lib):
    """What the kernels cover is a status code at the boundary, not a wrong result: TurboQuantProd pages
    come with 8 KV heads of dimension 128 and at most 64 query heads (the kernel stages 8 heads per token
    row); the query group is at most 16 heads; the staged TQ4 kernel (the one that rotates the query
    itself) serves KV heads of dimension 128 in groups of 8 and every other shape runs the direct kernel."""
    f = lib.fq_prod_paged_decode
    f.argtypes = ([ctypes.c_void_p] * 7 + [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p] + [ctypes.c_int] * 6 +
                  [ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t,
                   ctypes.c_void_p])

    def prod(S=2, HQ=32, HKV=8, D=128, BS=16, MB=4, NB=64, dtype=1, ptr=0):
        return f(_p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), _p(ptr), 0, _p(ptr), _p(ptr), S, HQ, HKV, D, BS,
                 MB, NB, 0.088, dtype, 0, _p(), 0, _p())

    assert prod(S=0) == FQ_OK
    assert prod(D=64) == FQ_DIM and prod(D=256) == FQ_DIM
    assert prod(HKV=4, HQ=16) == FQ_SHAPE
    assert prod(HQ=128) == FQ_SHAPE           # more than 8 query heads per KV head
    assert prod(HQ=8 * 17) == FQ_SHAPE
    assert prod(HKV=12, HQ=24) == FQ_SHAPE    # KV heads come in groups of 8
    assert prod(HKV=16, HQ=128) == FQ_NULL and prod(HKV=32, HQ=32) == FQ_NULL
    assert prod() == FQ_NULL                  # a supported shape gets as far as the pointer check
    lib.fq_paged_decode_fuses_rotation.argtypes = [ctypes.c_int] * 3
    assert lib.fq_paged_decode_fuses_rotation(128, 8, 1) == 1
    assert lib.fq_paged_decode_fuses_rotation(128, 16, 1) == 1 and lib.fq_paged_decode_fuses_rotation(128, 40, 1) == 1
    for d, hkv in ((64, 8), (256, 8), (128, 4), (128, 12), (128, 2)):
        assert lib.fq_paged_decode_fuses_rotation(d, hkv, 1) == 0
    # a pre-rotated query with a rotation matrix is only accepted where the kernel rotates it
    g = lib.fq_paged_tq4_decode
    g.argtypes = ([ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int] + [ctypes.c_void_p] * 8 + [ctypes.c_int] * 6 +
                  [ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_int, ctypes.c_void_p])
    assert g(_p(4096), _p(4096), 0, *([_p(4096)] * 8), 2, 16, 4, 128, 16, 4, 64, 0.088, 1, 1, _p()) == FQ_SHAPE
