"""The vLLM attention-backend plugin (src/flashquant/vllm/): the page-size arithmetic of the cache
spec and the kernel calls of the attention implementation import without vLLM; the backend, the
implementation class and the spec class derive from vLLM's own and are built on first use;
``register_flashquant_backend`` hooks them into a running vLLM."""
from flashquant_amd.vllm.backend import get_flashquant_backend_class
from flashquant_amd.vllm.compat import VLLM_MAX, VLLM_MIN, check_vllm_version
from flashquant_amd.vllm.impl import TQ4AttentionKernels, get_flashquant_impl_class
from flashquant_amd.vllm.registration import register_flashquant_backend
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
    "register_flashquant_backend", "get_flashquant_backend_class", "get_flashquant_impl_class", "check_vllm_version",
    "VLLM_MIN", "VLLM_MAX", "TQ4AttentionKernels", "TQ4_NORM_BYTES", "get_flashquant_attention_spec", "get_kv_cache_shape",
    "prod_bytes_per_token_kv", "prod_kv_cache_shape", "real_page_size_bytes", "tq4_bytes_per_token",
    "tq4_bytes_per_token_kv", "tq4_row_offsets",
]
