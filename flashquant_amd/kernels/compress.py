"""TQ4 compress operator (signature of src/flashquant/kernels/compress.py:50-95)."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from flashquant_amd.kernels._native import native, require_gpu


def tq4_compress(
    x: torch.Tensor,
    rotation: torch.Tensor,
    boundaries: torch.Tensor,
    *,
    rotation_T_even: Optional[torch.Tensor] = None,
    rotation_T_odd: Optional[torch.Tensor] = None,
    out: Optional[Tuple[torch.Tensor, torch.Tensor]] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Compress ``x`` (N, H, D) fp16/bf16 to nibble-packed TQ4.

    Returns ``(packed (N, H, D//2) uint8, norms (N, H, 1) float32)``.  The
    kernel takes rotation.T split into even and odd columns; they are derived
    from ``rotation`` when not supplied, as the reference's dispatcher does.
    """
    require_gpu(x, "x")
    if rotation_T_even is None or rotation_T_odd is None:
        rot_t = rotation.T.contiguous()
        rotation_T_even = rot_t[:, 0::2].contiguous()
        rotation_T_odd = rot_t[:, 1::2].contiguous()
    return native().tq4_compress(x, rotation_T_even, rotation_T_odd, boundaries, out)


def tq4_compress_and_store(
    key: torch.Tensor,
    value: torch.Tensor,
    rotation: torch.Tensor,
    boundaries: torch.Tensor,
    kv_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    *,
    rotation_T_even: Optional[torch.Tensor] = None,
    rotation_T_odd: Optional[torch.Tensor] = None,
) -> None:
    """Compress ``key`` and ``value`` (N, H, D) and write each token's packed row
    ``[K idx | K norms | V idx | V norms]`` into ``kv_cache`` (num_blocks,
    block_size, H*(D+8)) at flat slot ``slot_mapping[i]``: the work of the
    reference's ``_compress_and_store`` (src/flashquant/vllm/impl.py:220-263) in
    one launch.  Tokens beyond ``len(slot_mapping)`` and negative slots are not
    stored."""
    require_gpu(key, "key")
    if rotation_T_even is None or rotation_T_odd is None:
        rot_t = rotation.T.contiguous()
        rotation_T_even = rot_t[:, 0::2].contiguous()
        rotation_T_odd = rot_t[:, 1::2].contiguous()
    native().tq4_compress_store(key, value, rotation_T_even, rotation_T_odd, boundaries, kv_cache, slot_mapping)
