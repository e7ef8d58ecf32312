"""The pieces of the reference's vLLM backend that do not need vLLM itself: the page-size
arithmetic of its cache spec and the kernel calls of its attention implementation
(src/flashquant/vllm/spec.py, backend.py:124-138, impl.py)."""
from flashquant_amd.vllm.impl import TQ4AttentionKernels
from flashquant_amd.vllm.spec import (
    TQ4_NORM_BYTES,
    get_flashquant_attention_spec,
    get_kv_cache_shape,
    prod_bytes_per_token_kv,
    prod_kv_cache_shape,
    real_page_size_bytes,
    tq4_bytes_per_token,
    tq4_bytes_per_token_kv,
    tq4_row_offsets,
)

__all__ = [
    "TQ4AttentionKernels", "TQ4_NORM_BYTES", "get_flashquant_attention_spec", "get_kv_cache_shape",
    "prod_bytes_per_token_kv", "prod_kv_cache_shape", "real_page_size_bytes", "tq4_bytes_per_token",
    "tq4_bytes_per_token_kv", "tq4_row_offsets",
]
