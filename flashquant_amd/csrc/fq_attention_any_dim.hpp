// Parameter block and launcher of the any-head-dimension fused TQ4 attention kernel
// (fq_attention_any_dim.hip), shared with the host entry points in fq_fused_attention.hip.
#pragma once

#include <stdint.h>

namespace fq {

struct AnyDimParams {
    const uint16_t* q;
    const uint8_t* k_packed;    // contiguous operands: (B, H_KV, N_KV, D/2)
    const float* k_norms;
    const uint8_t* v_packed;
    const float* v_norms;
    const float* centroids_k;
    const float* centroids_v;
    const float* rotation;
    uint16_t* out;
    int rot_col_major;
    int H_Q, H_KV, G, N_Q, N_KV;
    int64_t k_cap, v_cap;       // tokens between the slabs of consecutive (batch, KV head) pairs (>= N_KV)
    int causal;
    float scale_log2e;
    const int32_t* cu_seqlens_q;   // paged operands
    const int32_t* seq_lens;
    const int32_t* block_table;
    const uint8_t* cache;
    int max_blocks, num_blocks, bs_log2;
};

// D in {64, 128, 256}; every argument already checked by the caller.
int launch_attention_any_dim(const AnyDimParams& p, int D, bool paged, int max_q, int batch, int dtype, void* stream);

}  // namespace fq

namespace fq_host {
// FQ_ATTENTION_ANY_DIM=1 routes head_dim 128 to the general kernel too (both are kept tested).
bool force_any_dim_attention();
}
