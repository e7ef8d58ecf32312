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
