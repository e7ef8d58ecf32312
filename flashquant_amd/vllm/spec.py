"""Page-size arithmetic of the packed KV cache (src/flashquant/vllm/spec.py:30-71,
src/flashquant/vllm/backend.py:124-138, byte offsets of src/flashquant/vllm/impl.py:132-138).

Plain functions, importable without vLLM; ``get_flashquant_attention_spec`` builds the
``FullAttentionSpec`` subclass on demand, as the reference does, and needs vLLM then."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

TQ4_NORM_BYTES = 4      # one float32 norm per head and per K / V
PROD_EXTRA_BYTES = 4    # TurboQuantProd keys carry a second float32, the residual norm


def tq4_bytes_per_token(head_dim: int) -> int:
    """Packed bytes of one token, one KV head, one of K or V: head_dim // 2 nibble-packed
    indices + a float32 norm (68 at head_dim 128)."""
    return head_dim // 2 + TQ4_NORM_BYTES


def tq4_bytes_per_token_kv(head_dim: int) -> int:
    """K and V together (136 at head_dim 128)."""
    return 2 * tq4_bytes_per_token(head_dim)


def tq4_row_offsets(num_kv_heads: int, head_dim: int) -> Tuple[int, int, int, int]:
    """(k_idx_end, k_norm_end, v_idx_end, total_bytes) of a token row
    ``[K idx | K norms | V idx | V norms]`` (src/flashquant/vllm/impl.py:132-138)."""
    half = head_dim // 2
    k_idx_end = num_kv_heads * half
    k_norm_end = k_idx_end + num_kv_heads * TQ4_NORM_BYTES
    v_idx_end = k_norm_end + num_kv_heads * half
    return k_idx_end, k_norm_end, v_idx_end, v_idx_end + num_kv_heads * TQ4_NORM_BYTES


def get_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int,
                       cache_dtype_str: str = "auto") -> Tuple[int, int, int]:
    """(num_blocks, block_size, num_kv_heads * (head_size + 8)) uint8
    (src/flashquant/vllm/backend.py:124-138)."""
    return num_blocks, block_size, num_kv_heads * tq4_bytes_per_token_kv(head_size)


def real_page_size_bytes(block_size: int, num_kv_heads: int, head_size: int) -> int:
    """What the block allocator provisions per page (src/flashquant/vllm/spec.py:60-66)."""
    return block_size * num_kv_heads * tq4_bytes_per_token_kv(head_size)


def prod_bytes_per_token_kv(head_dim: int) -> int:
    """TurboQuantProd keys (3-bit index + sign bit per coordinate, norm, residual norm) with TQ4
    values: head_dim + 12 bytes per token per KV head (140 at head_dim 128).  The reference has no
    page format for TurboQuantProd; this is the record of ``fq_prod_paged_decode``."""
    return tq4_bytes_per_token_kv(head_dim) + PROD_EXTRA_BYTES


def prod_kv_cache_shape(num_blocks: int, block_size: int, num_kv_heads: int, head_size: int) -> Tuple[int, int, int]:
    return num_blocks, block_size, num_kv_heads * prod_bytes_per_token_kv(head_size)


_spec_class = None


def get_flashquant_attention_spec() -> type:
    """``FlashQuantAttentionSpec``: vLLM's ``FullAttentionSpec`` with ``real_page_size_bytes``
    of the packed format (src/flashquant/vllm/spec.py:47-84).  Raises ImportError without vLLM."""
    global _spec_class
    if _spec_class is None:
        from vllm.v1.kv_cache_interface import FullAttentionSpec

        @dataclass(frozen=True, kw_only=True)
        class FlashQuantAttentionSpec(FullAttentionSpec):  # type: ignore[misc]
            @property
            def real_page_size_bytes(self) -> int:
                return real_page_size_bytes(self.block_size, self.num_kv_heads, self.head_size)

        _spec_class = FlashQuantAttentionSpec
    return _spec_class
