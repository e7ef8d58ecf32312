"""The attention backend class vLLM's registry instantiates (src/flashquant/vllm/backend.py:84-167).

The class derives from vLLM's FlashAttentionBackend and is therefore built on first use, when vLLM
can be imported: it declares the packed 3-D cache shape (num_blocks, block_size, H * (D + 8)) uint8,
names the implementation class and a metadata builder that allows graph capture of single-token
decode steps (the decode entry points of this library allocate nothing and synchronise nothing)."""
from __future__ import annotations

from typing import Tuple

from flashquant_amd.vllm.spec import get_kv_cache_shape as packed_cache_shape

_backend_class = None


def _vllm_flash_classes():
    from vllm.v1.attention.backends.flash_attn import FlashAttentionBackend, FlashAttentionMetadataBuilder
    return FlashAttentionBackend, FlashAttentionMetadataBuilder


def _make_metadata_builder():
    _, base = _vllm_flash_classes()

    class FlashQuantMetadataBuilder(base):  # type: ignore[misc, valid-type]
        @classmethod
        def get_cudagraph_support(cls, vllm_config, kv_cache_spec):
            from vllm.v1.attention.backend import AttentionCGSupport
            return AttentionCGSupport.UNIFORM_SINGLE_TOKEN_DECODE

    return FlashQuantMetadataBuilder


def _make_backend():
    base, _ = _vllm_flash_classes()
    builder = _make_metadata_builder()

    class FlashQuantAttentionBackend(base):  # type: ignore[misc, valid-type]
        """Packed TQ4 KV cache: nibble-packed indices and float32 norms as raw bytes."""

        # forward() writes the new tokens into the cache itself
        forward_includes_kv_cache_update = True

        @classmethod
        def supports_mm_prefix(cls) -> bool:
            return True

        @staticmethod
        def get_name() -> str:
            return "CUSTOM"            # the slot of AttentionBackendEnum the plugin registers under

        @staticmethod
        def get_impl_cls():
            from flashquant_amd.vllm.impl import get_flashquant_impl_class
            return get_flashquant_impl_class()

        @staticmethod
        def get_builder_cls():
            return builder

        @staticmethod
        def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                               cache_dtype_str: str = "auto") -> Tuple[int, ...]:
            return packed_cache_shape(num_blocks, block_size, num_kv_heads, head_size, cache_dtype_str)

        @staticmethod
        def get_kv_cache_stride_order(include_num_layers_dimension: bool = False) -> Tuple[int, ...]:
            # vLLM falls back to the identity order, which the 3-D packed layout needs
            raise NotImplementedError

    return FlashQuantAttentionBackend


def get_flashquant_backend_class() -> type:
    """FlashQuantAttentionBackend, created on first call (needs vLLM)."""
    global _backend_class
    if _backend_class is None:
        _backend_class = _make_backend()
    return _backend_class
