"""CPU-only checks of the Python layer: the native module loads, exposes the
operator names the reference's dispatch layer probes for, and refuses CPU
tensors instead of falling back."""
from __future__ import annotations

import inspect

import pytest
import torch

import flashquant_amd
from flashquant_amd import kernels as K


def test_native_module_exposes_reference_operator_names():
    C = flashquant_amd.load_native()
    # names probed with hasattr(_C, ...) in src/flashquant/kernels/*.py and src/flashquant/vllm/impl.py:57
    for name in ("tq4_compress", "tq4_decompress", "split_k_paged_decode", "fused_paged_tq4_decode"):
        assert callable(getattr(C, name))
    assert C.abi_version == 1


def test_operator_signatures_match_the_reference_layer():
    # src/flashquant/kernels/compress.py:50-58, decompress.py:48-54, paged_decode.py:55-69
    assert list(inspect.signature(K.tq4_compress).parameters) == [
        "x", "rotation", "boundaries", "rotation_T_even", "rotation_T_odd", "out"]
    assert list(inspect.signature(K.tq4_decompress).parameters) == ["packed", "norms", "centroids", "dtype", "out"]
    assert list(inspect.signature(K.split_k_paged_decode).parameters) == [
        "q", "kv_cache", "block_table", "seq_lens", "centroids_k", "centroids_v", "rotation", "num_kv_heads",
        "head_dim", "block_size", "sm_scale", "out", "num_splits"]
    assert inspect.signature(K.tq4_decompress).parameters["dtype"].default == torch.float16
    assert inspect.signature(K.split_k_paged_decode).parameters["num_splits"].default == 0


def test_no_cpu_fallback():
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        K.tq4_decompress(torch.zeros(1, 1, 64, dtype=torch.uint8), torch.zeros(1, 1, 1), torch.zeros(16))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        K.tq4_compress(torch.zeros(1, 1, 128, dtype=torch.bfloat16), torch.eye(128), torch.zeros(15))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        K.split_k_paged_decode(torch.zeros(1, 8, 128, dtype=torch.bfloat16), torch.zeros(1, 16, 1088, dtype=torch.uint8),
                               torch.zeros(1, 1, dtype=torch.int32), torch.zeros(1, dtype=torch.int32),
                               torch.zeros(16), torch.zeros(16), torch.eye(128), 8, 128, 16)
    C = flashquant_amd.load_native()
    with pytest.raises(ValueError, match="GPU"):
        C.tq4_decompress(torch.zeros(1, 1, 64, dtype=torch.uint8), torch.zeros(1, 1, 1), torch.zeros(16),
                         torch.float16, None)


def test_names_the_reference_calls_with_cpu_tensors_are_not_exported():
    """The reference's core modules call _C.quantize / dequantize / nibble_pack / nibble_unpack with
    CPU tensors and no device test as soon as the names exist (src/flashquant/core/quantizer.py:43,
    140-143, 176-179; core/packing.py:37, 75, 94).  A GPU-only module must therefore not carry them at
    top level; the kernel operators, which the reference gates on .is_cuda, are there."""
    C = flashquant_amd.load_native()
    for name in ("quantize", "dequantize", "nibble_pack", "nibble_unpack"):
        assert not hasattr(C, name), name
    for name in ("mse_quantize", "mse_dequantize", "tq4_compress", "tq4_decompress", "fused_tq_attention",
                 "split_k_paged_decode", "fused_paged_tq4_decode"):
        assert hasattr(C, name), name
    for name in ("nibble_pack", "nibble_unpack", "pack_2bit", "unpack_2bit", "validate_indices"):
        assert hasattr(C.packing, name), name
    # the one set-up entry the reference calls on the host works on the host
    c, b = C.codebook.solve_lloyd_max(128, 4)
    assert c.device.type == "cpu" and c.shape == (16,) and b.shape == (15,)


def test_product_does_not_import_the_oracle():
    import os
    root = os.path.dirname(os.path.abspath(flashquant_amd.__file__))
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "tq_oracle" not in text and "import oracle" not in text and "from oracle" not in text, f


# ---- host set-up of the product against the oracle ---------------------------------------

@pytest.mark.parametrize("dim", [64, 128, 256])
@pytest.mark.parametrize("bits", [1, 2, 3, 4])
def test_codebook_solver_equals_the_oracle(dim, bits):
    from flashquant_amd import core
    from oracle import tq_oracle as O
    c, b = core.solve_lloyd_max(dim, bits)
    oc, ob = O.lloyd_max_gaussian(dim, bits)
    assert c.dtype == torch.float32 and c.shape == (1 << bits,) and b.shape == ((1 << bits) - 1,)
    assert torch.equal(c, oc)
    # the middle boundary is the mean of two opposite levels: zero up to the last bit of the doubles
    assert (b - ob).abs().max().item() < 1e-12


def test_codebook_registry_and_value_quantizer():
    from flashquant_amd import core
    reg = core.CodebookRegistry()
    cb = reg.get(128, 4)
    assert reg.get(128, 4) is cb and cb.bits == 4 and cb.dim == 128
    x = torch.tensor([-1.0, 0.0, float(cb.boundaries[3]), 1.0])
    idx = cb.quantize(x)
    assert idx.tolist() == [0, int((cb.boundaries < 0).sum()), 3, 15]          # a tie goes to the lower cell
    assert torch.equal(cb.dequantize(idx), cb.centroids[idx])
    reg.clear()
    assert reg.get(128, 4) is not cb


@pytest.mark.parametrize("dim,seed", [(128, 42), (128, 43), (64, 42), (256, 5)])
def test_rotation_and_sketch_equal_the_oracle(dim, seed):
    from flashquant_amd import core
    from oracle import tq_oracle as O
    r = core.haar_orthogonal(dim, seed)
    assert torch.equal(r, O.haar_orthogonal(dim, seed))
    assert torch.equal(core.qjl_matrix(dim, seed), O.qjl_matrix(dim, seed))
    e, o = core.split_rotation(r)
    oe, oo = O.split_rotation(r)
    assert torch.equal(e, oe) and torch.equal(o, oo) and e.is_contiguous()


def test_quantizer_classes_hold_reference_state_and_refuse_cpu_tensors():
    from flashquant_amd import core
    from oracle import tq_oracle as O
    q = core.TurboQuantProd(128, 4, seed=42)
    assert q.mse_quantizer.bits == 3 and q.qjl_dim == 128
    assert torch.equal(q.mse_quantizer.rotation, O.haar_orthogonal(128, 42))
    assert torch.equal(q.qjl_matrix, O.qjl_matrix(128, 42))
    with pytest.raises(ValueError):
        core.TurboQuantProd(128, 1)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        q.quantize(torch.zeros(2, 128))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        core.TurboQuantMSE(64, 2).dequantize(torch.zeros(2, 64, dtype=torch.long), torch.ones(2, 1))
    assert core.KeyCompressor(128).quantizer.mse_quantizer.bits == 3
    assert torch.equal(core.ValueCompressor(128).quantizer.rotation, O.haar_orthogonal(128, 43))


# ---- page-size arithmetic of the serving backend (no vLLM needed) -------------------------------

def test_cache_spec_arithmetic_matches_the_reference_formulas():
    from flashquant_amd import vllm as V
    # src/flashquant/vllm/spec.py:30-44: head_dim // 2 + 4 per K or V; twice that per token and head
    assert V.TQ4_NORM_BYTES == 4
    assert V.tq4_bytes_per_token(128) == 68 and V.tq4_bytes_per_token_kv(128) == 136
    assert V.tq4_bytes_per_token(64) == 36 and V.tq4_bytes_per_token_kv(256) == 264
    # src/flashquant/vllm/impl.py:132-138
    assert V.tq4_row_offsets(8, 128) == (512, 544, 1056, 1088)
    assert V.tq4_row_offsets(2, 64) == (64, 72, 136, 144)
    # src/flashquant/vllm/backend.py:124-138, spec.py:60-66
    assert V.get_kv_cache_shape(1000, 16, 8, 128) == (1000, 16, 1088)
    assert V.real_page_size_bytes(16, 8, 128) == 17408
    # the compression ratio the reference logs: fp16 K and V against the packed row (3.76x)
    assert abs(2 * 8 * 128 * 2 / V.tq4_row_offsets(8, 128)[3] - 3.7647) < 1e-3
    # TurboQuantProd pages of this library: 12 more bytes per head than head_dim
    assert V.prod_bytes_per_token_kv(128) == 140 and V.prod_kv_cache_shape(10, 16, 8, 128) == (10, 16, 1120)
    from oracle import tq_oracle as O
    assert O.page_layout(8, 128) == V.tq4_row_offsets(8, 128)
    assert O.prod_page_layout(8, 128)[4] == 8 * V.prod_bytes_per_token_kv(128)
    with pytest.raises(ImportError):
        V.get_flashquant_attention_spec()            # vLLM is not installed here


def test_quantizer_and_codebook_class_surface_on_the_host():
    """_C.codebook / _C.quantizer carry the classes of the reference's C++ bindings
    (csrc/bindings/codebook_bind.cpp:11-49, quantizer_bind.cpp:10-64); construction and the
    codebook helpers run on the host."""
    from oracle import tq_oracle as O
    C = flashquant_amd.load_native()
    cb = C.codebook.LloydMaxCodebook(128, 4)
    c, b = O.lloyd_max_gaussian(128, 4)
    assert cb.dim == 128 and cb.bits == 4 and torch.equal(cb.centroids, c) and torch.allclose(cb.boundaries, b, atol=1e-12)
    x = torch.tensor([-1.0, -0.01, 0.0, 0.3, 1.0])
    # (the middle boundary is 0 up to 1e-16 on either side: compare on this codebook's own values)
    assert torch.equal(C.codebook.quantize(x, cb.boundaries), torch.bucketize(x, cb.boundaries))
    assert C.codebook.quantize(torch.tensor([-1.0, -0.01, 0.3, 1.0]), cb.boundaries).tolist() == [0, 7, 15, 15]
    idx = torch.tensor([[0, 5], [15, 8]])
    assert torch.equal(C.codebook.dequantize(idx, cb.centroids), c[idx])
    reg = C.codebook.CodebookRegistry.instance()
    got = reg.get(64, 3, torch.device("cpu"))
    assert got.bits == 3 and got.centroids.shape == (8,) and torch.equal(got.centroids, O.lloyd_max_gaussian(64, 3)[0])
    reg.warmup([128], [2, 4], torch.device("cpu"))
    reg.clear()
    q = C.quantizer.TurboQuantMSE(128, 4, 42)
    assert q.dim == 128 and q.bits == 4 and torch.equal(q.rotation(), O.haar_orthogonal(128, 42))
    p = C.quantizer.TurboQuantProd(128, 4)
    assert p.dim == 128 and p.bits == 4 and torch.equal(p.qjl_matrix(), O.qjl_matrix(128, 42))
    with pytest.raises(ValueError):
        C.quantizer.TurboQuantProd(128, 1)
    with pytest.raises(ValueError, match="GPU"):
        q.quantize(torch.zeros(2, 128))
    for name in ("QuantizedMSE", "QuantizedProd"):
        assert hasattr(C.quantizer, name)
