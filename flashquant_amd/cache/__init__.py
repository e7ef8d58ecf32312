"""Pre-allocated compressed KV storage for the fused attention path
(counterpart of src/flashquant/cache/buffer_pool.py)."""
from flashquant_amd.cache.buffer_pool import CompressedBuffer, CompressedKVLayer

__all__ = ["CompressedBuffer", "CompressedKVLayer"]
