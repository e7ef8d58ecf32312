"""Pre-allocated buffers for nibble-packed TQ4 indices and norms on the GPU.

``CompressedBuffer`` has the interface of the reference's ring buffer
(src/flashquant/cache/buffer_pool.py:21-140): ``append`` writes at the current
length, ``get`` returns views of the valid part without copying, an append past
the capacity raises ``RuntimeError``.  Two things are added for the fused path:
``append_from`` compresses new rows straight into the buffer (one launch, no
intermediate tensors), and the views ``get`` returns go into
``flashquant_amd.kernels.fused_tq_attention`` as they are, strided, so a decode
step neither decompresses nor copies the cache (the "fused mode" of the
reference's HF cache, src/flashquant/cache/hf_cache.py:322-329, 387-414).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from flashquant_amd.kernels._native import native, require_gpu


class CompressedBuffer:
    """(batch, heads, max_seq, half_dim) uint8 indices and (batch, heads, max_seq, 1)
    float32 norms, filled from position 0."""

    def __init__(self, max_seq: int, batch: int, heads: int, half_dim: int,
                 dtype: torch.dtype = torch.uint8, device: Optional[torch.device] = None) -> None:
        if device is None:
            device = torch.device("cuda")
        self.max_seq = max_seq
        self.batch = batch
        self.heads = heads
        self.half_dim = half_dim
        self._indices = torch.empty(batch, heads, max_seq, half_dim, dtype=dtype, device=device)
        self._norms = torch.empty(batch, heads, max_seq, 1, dtype=torch.float32, device=device)
        self._len = 0

    def _check_room(self, new_tokens: int) -> int:
        end = self._len + new_tokens
        if end > self.max_seq:
            raise RuntimeError(
                f"CompressedBuffer overflow: appending {new_tokens} tokens at position {self._len} "
                f"would exceed max_seq={self.max_seq}. Increase FlashQuantConfig.max_seq_len.")
        return end

    def append(self, indices: torch.Tensor, norms: torch.Tensor) -> None:
        """Write already compressed tokens ``(batch, heads, new_tokens, half_dim)`` /
        ``(batch, heads, new_tokens, 1)`` at the current position."""
        end = self._check_room(indices.shape[2])
        self._indices[:, :, self._len:end, :] = indices
        self._norms[:, :, self._len:end, :] = norms
        self._len = end

    def append_from(self, x: torch.Tensor, rot_T_even: torch.Tensor, rot_T_odd: torch.Tensor,
                    boundaries: torch.Tensor) -> None:
        """Compress ``x`` (batch, heads, new_tokens, 2 * half_dim), float16 or bfloat16, and
        write it at the current position in one launch.  ``rot_T_even`` / ``rot_T_odd`` are
        ``rotation.T[:, 0::2]`` / ``rotation.T[:, 1::2]`` (``_C.split_rotation``)."""
        require_gpu(x, "x")
        end = self._check_room(x.shape[2])
        native().tq4_compress_append(x, rot_T_even, rot_T_odd, boundaries, self._indices, self._norms, self._len)
        self._len = end

    def get(self) -> Tuple[torch.Tensor, torch.Tensor]:
        """Views of the valid part: ``(batch, heads, length, half_dim)`` and
        ``(batch, heads, length, 1)``."""
        return self._indices[:, :, :self._len, :], self._norms[:, :, :self._len, :]

    @property
    def length(self) -> int:
        return self._len

    def reset(self) -> None:
        self._len = 0


class CompressedKVLayer:
    """Keys and values of one attention layer in two ``CompressedBuffer`` objects, with the
    operations of a fused-mode cache step: ``update`` compresses and appends the new keys and
    values, ``attend`` runs the fused TQ4 attention over everything stored so far."""

    def __init__(self, max_seq: int, batch: int, heads: int, head_dim: int, rotation: torch.Tensor,
                 centroids: torch.Tensor, boundaries: torch.Tensor, device: Optional[torch.device] = None) -> None:
        if device is None:
            device = torch.device("cuda")
        self.keys = CompressedBuffer(max_seq, batch, heads, head_dim // 2, device=device)
        self.values = CompressedBuffer(max_seq, batch, heads, head_dim // 2, device=device)
        self.rotation = rotation.to(device)
        self.centroids = centroids.to(device)
        self.boundaries = boundaries.to(device)
        ev, od = native().split_rotation(rotation.cpu())
        self._rot_T_even, self._rot_T_odd = ev.to(device), od.to(device)

    def update(self, key_states: torch.Tensor, value_states: torch.Tensor) -> None:
        """``key_states``, ``value_states`` (batch, heads, new_tokens, head_dim)."""
        self.keys.append_from(key_states, self._rot_T_even, self._rot_T_odd, self.boundaries)
        self.values.append_from(value_states, self._rot_T_even, self._rot_T_odd, self.boundaries)

    def get_compressed(self):
        """(k_packed, k_norms, v_packed, v_norms), views (the reference's ``get_compressed``,
        src/flashquant/cache/hf_cache.py:387-414)."""
        return (*self.keys.get(), *self.values.get())

    def attend(self, q: torch.Tensor, sm_scale: Optional[float] = None, is_causal: bool = False) -> torch.Tensor:
        from flashquant_amd.kernels import fused_tq_attention
        kp, kn, vp, vn = self.get_compressed()
        return fused_tq_attention(q, kp, kn, vp, vn, self.centroids, self.centroids, self.rotation, sm_scale, is_causal)

    @property
    def length(self) -> int:
        return self.keys.length
