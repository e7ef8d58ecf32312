"""Operator layer with the signatures of the reference's ``flashquant.kernels``
(src/flashquant/kernels/__init__.py): tq4_compress, tq4_decompress,
fused_tq_attention, split_k_paged_decode.  Every call goes to the HIP kernels
through ``flashquant_amd._C``; nothing here computes on the CPU."""
from flashquant_amd.kernels.attention import fused_tq_attention, paged_tq4_prefill
from flashquant_amd.kernels.compress import tq4_compress, tq4_compress_and_store
from flashquant_amd.kernels.decompress import tq4_decompress, tq4_decompress_rotated
from flashquant_amd.kernels.packing import nibble_pack, nibble_unpack, pack_2bit, unpack_2bit
from flashquant_amd.kernels.paged_decode import split_k_paged_decode, tq4_store_and_decode
from flashquant_amd.kernels.prod import prod_compress, prod_paged_decode, prod_page_layout, prod_store_rows

__all__ = ["tq4_compress", "tq4_compress_and_store", "tq4_decompress", "tq4_decompress_rotated", "fused_tq_attention", "paged_tq4_prefill", "split_k_paged_decode", "tq4_store_and_decode", "nibble_pack", "nibble_unpack", "pack_2bit", "unpack_2bit",
           "prod_compress", "prod_paged_decode", "prod_page_layout", "prod_store_rows"]
