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


def test_product_does_not_import_the_oracle():
    import os
    root = os.path.dirname(os.path.abspath(flashquant_amd.__file__))
    for dirpath, _, files in os.walk(root):
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".hpp", ".h")):
                text = open(os.path.join(dirpath, f), errors="ignore").read()
                assert "tq_oracle" not in text and "import oracle" not in text and "from oracle" not in text, f
