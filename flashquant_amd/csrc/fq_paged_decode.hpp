// Shared by the split-K paged decode kernels: the launch parameters, the chunk sizing of ragged
// long-context batches and the launch helper.
#pragma once

#include "fq_common.hpp"
#include "fq_device.hpp"

namespace fq {

struct DecodeParams {
    const void* q_rot;          // (S, H_Q, D) query dtype: rotated, or un-rotated when `rotation` is set
    int rot_col_major;          // layout of `rotation` / of the matrix given to the side kernels
    const float* rotation;      // staged kernel only: rotate the query in the prologue (NULL: already rotated)
    const float* sketch;        // TurboQuantProd pages only: the (D, D) sign-sketch matrix S
    const uint8_t* cache;       // (num_blocks, BS, H_KV*(D+8))
    const int32_t* block_table; // (S, max_blocks)
    const int32_t* seq_lens;    // (S,)
    const float* centroids_k;
    const float* centroids_v;
    float* part_acc;            // (S, H_Q, NS, D)
    float* part_m;              // (S, H_Q, NS)
    float* part_l;              // (S, H_Q, NS)
    int H_Q, H_KV, G;           // G = H_Q / H_KV
    int max_blocks;
    int num_blocks;
    int num_splits;
    int two_tables;             // centroids_v differs from centroids_k
    float scale_log2e;          // sm_scale * log2(e)
    int heads_per_wg;           // direct kernel: KV heads a workgroup serves; its other wavefronts take further splits
    int spin_limit;             // staged kernel: polls of a bounded wait between wavefronts before it gives up
    int balance_slots;          // staged kernel: > 0 lets the workgroups size the token chunks from the actual
                                // sequence lengths, for this many workgroups running at a time (num_seqs <= 64)
    // Staged kernel instantiated with STORE: the serving step in one launch.  The workgroup whose split
    // holds a sequence's last token first compresses that token's new key and value rows into their
    // cache row (slot new_slots[seq]; negative: not stored), then reads the row back with its tile.
    uint8_t* cache_rw;          // the cache again, for the row that is written
    const void* new_key;        // (S, H_KV, D) query dtype, one token per sequence
    const void* new_value;
    const int64_t* new_slots;   // (S,) flat slot of the new token
    const float* boundaries;    // (15,) ascending
    int64_t num_slots;          // num_blocks * block_size
};


// Ragged batches of long contexts (at most 64 sequences, one lane each).  With the chunk
// of the longest possible context the live workgroups are all the same size and their
// count is whatever the lengths add up to, e.g. 2.1 rounds over the chip, which costs 3.
// Every workgroup evaluates the same 64 candidate chunk sizes (one per lane) on the
// actual lengths, cost = rounds x (chunk + a prologue's worth of tokens), and takes the
// cheapest: same inputs, same arithmetic, same answer in every workgroup.  Larger chunks
// only: the split count bounds the chunk from below.  On return `chunk` is the chosen size,
// (`seq`, `split`) the pair this workgroup takes and `L_known` its sequence's length.
// TPR: tokens per row of the kernel (rows of 2, 4 or 8 consecutive tokens when the model has 4, 2 or 1 KV heads)
template <int PVR, int BS, int TPR>
__device__ __forceinline__ void balance_chunks(const DecodeParams& p, int lane, int NS, bool rowwide, int& chunk, int& seq,
                                               int& split, int& L_known) {
    const int cap = rowwide ? chunk * NS : 64 * PVR * BS;       // page ids of a split: 64 * PVR lanes
    const int step = ((chunk >> 4) + 63) & ~63;
    int cand = chunk + lane * step;
    cand = cand < cap ? cand : cap;
    cand = cand > chunk ? cand : chunk;
    const float rc = __builtin_amdgcn_rcpf(float(cand));
    const int nseq = int(gridDim.x);
    int l_real = lane < nseq ? p.seq_lens[lane] : 0;
    l_real = l_real < 0 ? 0 : (l_real > p.max_blocks * BS * TPR ? p.max_blocks * BS * TPR : l_real);
    const int l_mine = (l_real + TPR - 1) / TPR;               // in rows
    float groups = 0.0f;
    for (int sq = 0; sq < nseq; ++sq)
        groups += __builtin_ceilf(float(__builtin_amdgcn_readlane(l_mine, sq)) * rc - 0.0009765625f);
    const float rounds = __builtin_ceilf(groups * __builtin_amdgcn_rcpf(float(p.balance_slots)) - 0.0009765625f);
    const float cost = (rounds < 1.0f ? 1.0f : rounds) * float(cand + 96);
    uint32_t key = (uint32_t(cost) << 6) | uint32_t(lane);
#pragma unroll
    for (int mask = 1; mask < 64; mask <<= 1) {
        const uint32_t other = uint32_t(__shfl_xor(int(key), mask, kWave));
        key = other < key ? other : key;
    }
    const int best = chunk + int(key & 63u) * step;
    chunk = best < cap ? best : (cap > chunk ? cap : chunk);

    // The live (sequence, split) pairs first, in sequence order, then the empty ones: the w-th
    // workgroup of the grid takes the w-th pair of that list.  Live workgroups are all of one
    // size and now consecutive, so they spread evenly over the XCDs and CUs whatever the lengths.
    auto scan = [&](int v) {
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int t = __shfl_up(v, d, kWave);
            v += lane >= d ? t : 0;
        }
        return v;
    };
    int n_mine = lane < nseq ? (l_mine + chunk - 1) / chunk : 0;
    n_mine = n_mine < NS ? n_mine : NS;
    const int live_incl = scan(n_mine);
    const int total_live = __builtin_amdgcn_readlane(live_incl, 63);
    const int w = int(blockIdx.x) + int(gridDim.x) * int(blockIdx.y);
    if (w < total_live) {
        const int s_idx = __builtin_popcountll(__ballot(live_incl <= w));
        seq = s_idx;
        split = w - __builtin_amdgcn_readlane(live_incl - n_mine, s_idx);
    } else {
        const int e = w - total_live;
        const int dead_mine = lane < nseq ? NS - n_mine : 0;
        const int dead_incl = scan(dead_mine);
        int s_idx = __builtin_popcountll(__ballot(dead_incl <= e));
        s_idx = s_idx < nseq ? s_idx : nseq - 1;
        seq = s_idx;
        split = __builtin_amdgcn_readlane(n_mine, s_idx) + (e - __builtin_amdgcn_readlane(dead_incl - dead_mine, s_idx));
        split = split < NS ? split : NS - 1;
    }
    L_known = __builtin_amdgcn_readlane(l_real, seq);
}

// Launch with `lds` bytes of dynamic LDS; more than 64 KB per workgroup has to be
// allowed per kernel function first.
template <typename K>
inline int launch_with_lds(K kernel, const DecodeParams& p, dim3 grid, dim3 block, size_t lds, hipStream_t stream) {
    if (lds > 32768 && !fq_host::lds_limit_raised(reinterpret_cast<const void*>(kernel), lds)) return FQ_ERR_LAUNCH;
    hipLaunchKernelGGL(kernel, grid, block, lds, stream, p);
    return fq_host::check_launch();
}

// The ring kernel (fq_paged_decode_ring.hip): groups of 8 KV heads of dimension 128, TQ4 pages.
int launch_ring(const DecodeParams& p, int num_seqs, int block_size, bool wide, int dtype, hipStream_t stream);

}  // namespace fq
