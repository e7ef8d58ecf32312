"""The vLLM plugin layer against a stand-in ``vllm`` package (vLLM itself is not installed here): the
version gate, the backend class, the registration steps and the dispatch of the implementation's
forward().  The reference tests the same surface against mocks (tests/test_vllm_impl.py:9-45,
tests/test_vllm_registration.py:9-63); the kernels behind it are covered on the GPU through
``TQ4AttentionKernels`` (tests/test_gpu_surface.py)."""
from __future__ import annotations

import enum
import sys
import types
from dataclasses import dataclass
from unittest.mock import MagicMock

import pytest
import torch

from flashquant_amd.errors import FlashQuantCompatError


def _install_fake_vllm(monkeypatch, version="0.20.1.dev0+rocm"):
    """A package with the handful of vLLM names the plugin touches; returns what the tests look at."""
    seen = {"registered": []}

    def module(name, **attrs):
        m = types.ModuleType(name)
        m.__dict__.update(attrs)
        monkeypatch.setitem(sys.modules, name, m)
        return m

    class FlashAttentionBackend:
        pass

    class FlashAttentionMetadataBuilder:
        pass

    class FlashAttentionImpl:
        def __init__(self, num_heads=32, head_size=128, scale=0.0884, num_kv_heads=8, attn_type="decoder"):
            self.num_heads, self.head_size, self.scale, self.num_kv_heads, self.attn_type = (
                num_heads, head_size, scale, num_kv_heads, attn_type)

        def _forward_encoder_attention(self, q, k, v, out, md, layer):
            return "encoder"

    class AttentionCGSupport(enum.Enum):
        NEVER = 0
        UNIFORM_SINGLE_TOKEN_DECODE = 1

    class AttentionType:
        DECODER, ENCODER, ENCODER_ONLY = "decoder", "encoder", "encoder_only"

    class AttentionBackendEnum(enum.Enum):
        FLASH_ATTN = 0
        CUSTOM = 1

    def register_backend(slot, path):
        seen["registered"].append((slot, path))

    @dataclass(frozen=True, kw_only=True)
    class FullAttentionSpec:
        block_size: int
        num_kv_heads: int
        head_size: int
        dtype: torch.dtype

    class Attention:
        def get_kv_cache_spec(self, vllm_config):
            return FullAttentionSpec(block_size=16, num_kv_heads=8, head_size=128, dtype=torch.bfloat16)

    spec_manager_map = {FullAttentionSpec: "full-attention manager"}
    module("vllm", __version__=version)
    for name in ("vllm.v1", "vllm.v1.attention", "vllm.v1.attention.backends", "vllm.v1.core", "vllm.model_executor",
                 "vllm.model_executor.layers", "vllm.model_executor.layers.attention"):
        module(name)
    module("vllm.v1.attention.backends.flash_attn", FlashAttentionBackend=FlashAttentionBackend,
           FlashAttentionMetadataBuilder=FlashAttentionMetadataBuilder, FlashAttentionImpl=FlashAttentionImpl)
    module("vllm.v1.attention.backend", AttentionCGSupport=AttentionCGSupport, AttentionType=AttentionType)
    module("vllm.v1.attention.backends.registry", AttentionBackendEnum=AttentionBackendEnum, register_backend=register_backend)
    module("vllm.v1.kv_cache_interface", FullAttentionSpec=FullAttentionSpec)
    module("vllm.v1.core.single_type_kv_cache_manager", spec_manager_map=spec_manager_map)
    module("vllm.model_executor.layers.attention.attention", Attention=Attention)
    module("vllm.config", get_current_vllm_config_or_none=lambda: None)
    seen.update(FullAttentionSpec=FullAttentionSpec, Attention=Attention, spec_manager_map=spec_manager_map,
                AttentionBackendEnum=AttentionBackendEnum, AttentionCGSupport=AttentionCGSupport,
                FlashAttentionBackend=FlashAttentionBackend, FlashAttentionImpl=FlashAttentionImpl)
    return seen


@pytest.fixture
def fresh_plugin(monkeypatch):
    """The plugin's lazily built classes and its registered flag start empty and are put back."""
    import flashquant_amd.vllm.backend as backend
    import flashquant_amd.vllm.impl as impl
    import flashquant_amd.vllm.registration as registration
    import flashquant_amd.vllm.spec as spec
    monkeypatch.setattr(backend, "_backend_class", None)
    monkeypatch.setattr(impl, "_impl_class", None)
    monkeypatch.setattr(spec, "_spec_class", None)
    monkeypatch.setattr(registration, "_registered", False)
    monkeypatch.setattr(registration, "_stock_get_kv_cache_spec", None)
    return types.SimpleNamespace(backend=backend, impl=impl, registration=registration, spec=spec)


def test_version_gate(monkeypatch):
    from flashquant_amd.vllm.compat import check_vllm_version, parse_version
    assert parse_version("0.20.1.dev0+rocm") == (0, 20, 1) and parse_version("0.18") == (0, 18)
    monkeypatch.setitem(sys.modules, "vllm", None)                 # import vllm -> ImportError
    with pytest.raises(FlashQuantCompatError, match="not installed"):
        check_vllm_version()
    for version, ok in (("0.17.9", False), ("0.18.0", True), ("0.21.3rc1", True), ("0.22.0", False), ("1.0.0", False)):
        monkeypatch.setitem(sys.modules, "vllm", types.SimpleNamespace(__version__=version))
        if ok:
            assert check_vllm_version() == version
        else:
            with pytest.raises(FlashQuantCompatError, match="0.18.0"):
                check_vllm_version()


def test_backend_class(monkeypatch, fresh_plugin):
    fake = _install_fake_vllm(monkeypatch)
    B = fresh_plugin.backend.get_flashquant_backend_class()
    assert B is fresh_plugin.backend.get_flashquant_backend_class()            # built once
    assert issubclass(B, fake["FlashAttentionBackend"])
    assert B.get_name() == "CUSTOM" and B.forward_includes_kv_cache_update and B.supports_mm_prefix()
    assert B.get_kv_cache_shape(100, 16, 8, 128) == (100, 16, 8 * 136)
    assert B.get_kv_cache_shape(7, 32, 4, 64, "auto") == (7, 32, 4 * 72)
    with pytest.raises(NotImplementedError):
        B.get_kv_cache_stride_order()
    builder = B.get_builder_cls()
    assert builder.get_cudagraph_support(None, None) is fake["AttentionCGSupport"].UNIFORM_SINGLE_TOKEN_DECODE
    assert issubclass(B.get_impl_cls(), fake["FlashAttentionImpl"])


def test_registration_steps_and_idempotence(monkeypatch, fresh_plugin):
    fake = _install_fake_vllm(monkeypatch)
    reg = fresh_plugin.registration
    stock = fake["Attention"].get_kv_cache_spec
    reg.register_flashquant_backend()
    reg.register_flashquant_backend()                                        # the second call does nothing
    assert fake["registered"] == [(fake["AttentionBackendEnum"].CUSTOM,
                                   "flashquant_amd.vllm.backend._make_backend.<locals>.FlashQuantAttentionBackend")]
    spec_class = fresh_plugin.spec.get_flashquant_attention_spec()
    assert issubclass(spec_class, fake["FullAttentionSpec"])
    assert fake["spec_manager_map"][spec_class] == "full-attention manager"
    assert fake["Attention"].get_kv_cache_spec is not stock
    spec = fake["Attention"]().get_kv_cache_spec(None)
    assert isinstance(spec, spec_class) and spec.dtype == torch.uint8
    assert spec.real_page_size_bytes == 16 * 8 * 136                          # what the block allocator provisions


def test_registration_refuses_an_unsupported_vllm(monkeypatch, fresh_plugin):
    fake = _install_fake_vllm(monkeypatch, version="0.17.0")
    with pytest.raises(FlashQuantCompatError):
        fresh_plugin.registration.register_flashquant_backend()
    assert fake["registered"] == [] and not fresh_plugin.registration._registered
    # a supported version whose internals are missing is a compatibility error too, not an ImportError
    _install_fake_vllm(monkeypatch)
    monkeypatch.setitem(sys.modules, "vllm.v1.attention.backends.registry", None)
    with pytest.raises(FlashQuantCompatError, match="internal"):
        fresh_plugin.registration.register_flashquant_backend()


def test_impl_forward_dispatch(monkeypatch, fresh_plugin):
    """forward(): new tokens are stored first, a batch of single-token queries runs the paged decode,
    anything longer the paged prefill, both on the first num_actual_tokens rows."""
    _install_fake_vllm(monkeypatch)
    kernels = MagicMock()
    monkeypatch.setattr(fresh_plugin.impl, "TQ4AttentionKernels", MagicMock(return_value=kernels))
    Impl = fresh_plugin.impl.get_flashquant_impl_class()
    impl = Impl(num_heads=32, head_size=128, scale=0.0884, num_kv_heads=8)
    fresh_plugin.impl.TQ4AttentionKernels.assert_called_once_with(8, 128, 0.0884, torch.device("cuda"))

    q, k, v = torch.randn(4, 32, 128), torch.randn(4, 8, 128), torch.randn(4, 8, 128)
    out = torch.ones(4, 32, 128)
    cache = torch.zeros(10, 16, 8 * 136, dtype=torch.uint8)
    with pytest.raises(ValueError):
        impl.forward(None, q, k, v, cache, MagicMock(), output=None)
    with pytest.raises(NotImplementedError):
        impl.forward(None, q, k, v, cache, MagicMock(), output=out, output_scale=torch.ones(1))
    assert impl.forward(None, q, k, v, cache, None, output=out) is out and float(out.abs().sum()) == 0.0   # profiling run

    md = MagicMock(num_actual_tokens=3, max_query_len=1, use_cascade=False)
    assert impl.forward(None, q, k, v, cache, md, output=out) is out
    kernels.compress_and_store.assert_called_once_with(k, v, cache, md.slot_mapping)
    (q_arg, cache_arg, table_arg, lens_arg), kw = kernels.decode.call_args
    assert q_arg.shape[0] == 3 and cache_arg is cache and table_arg is md.block_table and lens_arg is md.seq_lens
    assert kw["out"].shape[0] == 3 and kw["out"].data_ptr() == out.data_ptr()
    kernels.prefill.assert_not_called()

    # a pure decode step (one new token per sequence): stored and attended over in one call
    md1 = MagicMock(num_actual_tokens=3, max_query_len=1, use_cascade=False, seq_lens=torch.tensor([5, 9, 1], dtype=torch.int32),
                    slot_mapping=torch.tensor([4, 40, 64, -1]))
    assert impl.forward(None, q, k, v, cache, md1, output=out) is out
    args, kw = kernels.decode_step.call_args
    assert [a.shape[0] for a in args[:3]] == [3, 3, 3] and args[3] is cache and args[4].tolist() == [4, 40, 64]
    assert args[4].dtype == torch.int64 and args[5] is md1.block_table and args[6] is md1.seq_lens
    assert kw["out"].shape[0] == 3 and kw["out"].data_ptr() == out.data_ptr()
    assert kernels.compress_and_store.call_count == 1 and kernels.decode.call_count == 1      # not called again

    md2 = MagicMock(num_actual_tokens=4, max_query_len=4, use_cascade=False, causal=True)
    impl.forward(None, q, None, None, cache, md2, output=out)                 # nothing new to store
    assert kernels.compress_and_store.call_count == 1
    args, kw = kernels.prefill.call_args
    assert args[0].shape[0] == 4 and args[1] is md2.query_start_loc and args[2] == 4 and args[3] is cache
    assert kw["causal"] is True and kw["out"].data_ptr() == out.data_ptr()

    md3 = MagicMock(num_actual_tokens=4, max_query_len=4, use_cascade=True)
    with pytest.raises(NotImplementedError):
        impl.forward(None, q, None, None, cache, md3, output=out)
    impl.attn_type = "encoder"
    assert impl.forward(None, q, k, v, cache, md2, output=out) == "encoder"
