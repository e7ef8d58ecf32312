"""The kernel calls of the reference's vLLM attention implementation, without vLLM.

``TQ4AttentionKernels`` holds what ``FlashQuantAttentionImpl.__init__`` sets up per layer
(src/flashquant/vllm/impl.py:100-162: rotation, codebook, the pre-split transposed rotation, the
byte offsets of a token row) and offers the four steps its ``forward`` is made of, each as one
launch of this library:

  compress_and_store   _compress_and_store, impl.py:220-263
  decode               _fused_decode_path, impl.py:362-394
  prefill              _tq4_prefill + flash_attn_varlen_func + post-rotation, impl.py:317-336, 470-512
  decompress_cache     _decompress_cache, impl.py:265-318

``get_flashquant_impl_class`` builds ``FlashQuantAttentionImpl``, the subclass of vLLM's
FlashAttentionImpl whose ``forward`` is these launches (needs vLLM, imported on first use); the rest
of the module imports without it."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from flashquant_amd.kernels._native import native, require_gpu
from flashquant_amd.vllm.spec import tq4_row_offsets

TQ4_BITS = 4
TQ4_SEED = 42        # the reference uses one rotation and one codebook for keys and values (impl.py:44-46)


class TQ4AttentionKernels:
    def __init__(self, num_kv_heads: int, head_size: int, scale: float, device: torch.device,
                 seed: int = TQ4_SEED) -> None:
        C = native()
        self.num_kv_heads = num_kv_heads
        self.head_size = head_size
        self.scale = float(scale)
        rotation = C.haar_orthogonal(head_size, seed)
        centroids, boundaries = C.codebook.solve_lloyd_max(head_size, TQ4_BITS)
        ev, od = C.split_rotation(rotation)
        self.rotation = rotation.to(device)
        self.centroids = centroids.to(device)
        self.boundaries = boundaries.to(device)
        self.rot_T_even = ev.to(device)
        self.rot_T_odd = od.to(device)
        self.k_idx_end, self.k_norm_end, self.v_idx_end, self.total_bytes = tq4_row_offsets(num_kv_heads, head_size)

    def compress_and_store(self, key: torch.Tensor, value: torch.Tensor, kv_cache: torch.Tensor,
                           slot_mapping: torch.Tensor) -> None:
        """``key``, ``value`` (tokens, H_KV, D); the rows of tokens ``i < len(slot_mapping)`` land in
        cache slot ``slot_mapping[i]``."""
        require_gpu(key, "key")
        native().tq4_compress_store(key, value, self.rot_T_even, self.rot_T_odd, self.boundaries, kv_cache, slot_mapping)

    def decode(self, query: torch.Tensor, kv_cache: torch.Tensor, block_table: torch.Tensor, seq_lens: torch.Tensor,
               out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """One query token per sequence, ``query`` (S, H_Q, D) un-rotated; original-space output."""
        require_gpu(query, "query")
        return native().fused_paged_tq4_decode(query, kv_cache, block_table, seq_lens, self.centroids, self.centroids,
                                               self.rotation, self.num_kv_heads, self.head_size, kv_cache.shape[1],
                                               sm_scale=self.scale, out=out)

    def decode_step(self, query: torch.Tensor, key: torch.Tensor, value: torch.Tensor, kv_cache: torch.Tensor,
                    slot_mapping: torch.Tensor, block_table: torch.Tensor, seq_lens: torch.Tensor,
                    out: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``compress_and_store`` of one new token per sequence followed by ``decode``, as one call
        (src/flashquant/vllm/impl.py:362-394): ``key`` / ``value`` (S, H_KV, D), ``slot_mapping`` (S,) int64,
        ``seq_lens`` counting the new token."""
        require_gpu(query, "query")
        return native().tq4_store_and_decode(key, value, slot_mapping, self.rot_T_even, self.rot_T_odd, self.boundaries,
                                             query, kv_cache, block_table, seq_lens, self.centroids, self.centroids,
                                             self.rotation, self.num_kv_heads, self.head_size, kv_cache.shape[1],
                                             sm_scale=self.scale, out=out)

    def prefill(self, query: torch.Tensor, query_start_loc: torch.Tensor, max_query_len: int, kv_cache: torch.Tensor,
                block_table: torch.Tensor, seq_lens: torch.Tensor, out: Optional[torch.Tensor] = None,
                causal: bool = True) -> torch.Tensor:
        """Variable-length prefill (or chunked prefill, or a mixed batch) straight from the packed
        cache; the new tokens must already be stored."""
        require_gpu(query, "query")
        return native().paged_tq4_prefill(query, query_start_loc, int(max_query_len), kv_cache, block_table, seq_lens,
                                          self.centroids, self.centroids, self.rotation, self.num_kv_heads,
                                          self.head_size, kv_cache.shape[1], self.scale, causal, out)

    def decompress_cache(self, kv_cache: torch.Tensor, compute_dtype: torch.dtype, *, apply_rotation: bool = True,
                         out_k: Optional[torch.Tensor] = None,
                         out_v: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """(key_cache, value_cache) of shape (NB, BS, H, D) in ``compute_dtype``: rotated space, or
        the original space with ``apply_rotation`` (then one launch per tensor does both steps)."""
        require_gpu(kv_cache, "kv_cache")
        C = native()
        nb, bs, _ = kv_cache.shape
        h, d = self.num_kv_heads, self.head_size
        flat = kv_cache.reshape(nb * bs, self.total_bytes)
        k_packed = flat[:, :self.k_idx_end].contiguous().reshape(-1, h, d // 2)
        k_norms = flat[:, self.k_idx_end:self.k_norm_end].contiguous().view(torch.float32).reshape(-1, h, 1)
        v_packed = flat[:, self.k_norm_end:self.v_idx_end].contiguous().reshape(-1, h, d // 2)
        v_norms = flat[:, self.v_idx_end:].contiguous().view(torch.float32).reshape(-1, h, 1)
        if apply_rotation:
            key_out = C.tq4_decompress_rotated(k_packed, k_norms, self.centroids, self.rotation, compute_dtype, out_k)
            value_out = C.tq4_decompress_rotated(v_packed, v_norms, self.centroids, self.rotation, compute_dtype, out_v)
        else:
            key_out = C.tq4_decompress(k_packed, k_norms, self.centroids, compute_dtype, out_k)
            value_out = C.tq4_decompress(v_packed, v_norms, self.centroids, compute_dtype, out_v)
        return key_out.reshape(nb, bs, h, d), value_out.reshape(nb, bs, h, d)


_impl_class = None


def _make_impl_class() -> type:
    from vllm.v1.attention.backends.flash_attn import FlashAttentionImpl

    class FlashQuantAttentionImpl(FlashAttentionImpl):  # type: ignore[misc, valid-type]
        """forward(): store the new tokens in the packed cache, then attend straight from it.

        Where the reference decompresses the whole cache and hands it to a FlashAttention library
        (src/flashquant/vllm/impl.py:395-512), a batch of single-token queries runs the split-K paged
        decode and everything else the paged prefill, both reading the packed pages; neither
        allocates, so a decode step can be captured in a graph."""

        def __init__(self, *args, **kwargs) -> None:
            super().__init__(*args, **kwargs)
            from vllm.config import get_current_vllm_config_or_none
            cfg = get_current_vllm_config_or_none()
            device = cfg.device_config.device if cfg is not None else torch.device("cuda")
            self._tq4 = TQ4AttentionKernels(self.num_kv_heads, self.head_size, self.scale, device)

        def forward(self, layer, query, key, value, kv_cache, attn_metadata, output=None, output_scale=None,
                    output_block_scale=None):
            if output is None:
                raise ValueError("FlashQuantAttentionImpl needs a pre-allocated output")
            if output_scale is not None or output_block_scale is not None:
                raise NotImplementedError("fused output quantisation is not supported by the FlashQuant backend")
            if attn_metadata is None:                       # profiling run
                output.zero_()
                return output
            from vllm.v1.attention.backend import AttentionType
            n = attn_metadata.num_actual_tokens
            if self.attn_type in (AttentionType.ENCODER_ONLY, AttentionType.ENCODER):
                return self._forward_encoder_attention(query[:n], key[:n], value[:n], output[:n], attn_metadata, layer)
            if getattr(attn_metadata, "use_cascade", False):
                raise NotImplementedError("cascade attention is not supported by the FlashQuant backend")
            slots = attn_metadata.slot_mapping
            if (attn_metadata.max_query_len == 1 and key is not None and value is not None
                    and n == attn_metadata.seq_lens.shape[0] and slots.shape[0] >= n):
                # a pure decode step: one new token per sequence, stored and attended over in one call
                self._tq4.decode_step(query[:n], key[:n], value[:n], kv_cache, slots[:n].long(), attn_metadata.block_table,
                                      attn_metadata.seq_lens, out=output[:n])
                return output
            if key is not None and value is not None:
                self._tq4.compress_and_store(key, value, kv_cache, slots)
            if attn_metadata.max_query_len == 1:
                self._tq4.decode(query[:n], kv_cache, attn_metadata.block_table, attn_metadata.seq_lens, out=output[:n])
            else:
                self._tq4.prefill(query[:n], attn_metadata.query_start_loc, attn_metadata.max_query_len, kv_cache,
                                  attn_metadata.block_table, attn_metadata.seq_lens, out=output[:n],
                                  causal=getattr(attn_metadata, "causal", True))
            return output

    return FlashQuantAttentionImpl


def get_flashquant_impl_class() -> type:
    """FlashQuantAttentionImpl, created on first call (needs vLLM)."""
    global _impl_class
    if _impl_class is None:
        _impl_class = _make_impl_class()
    return _impl_class
