// Fused TQ4 FlashAttention (prefill) for gfx950, head_dim 64 and 128: un-rotated query in,
// packed TQ4 keys and values in, original-space output out.  (The figures in this comment are
// those of head_dim 128.)
//
// Operator: fused_tq_attention_reference
// (src/flashquant/kernels/cpu_reference.py:154-227) as dispatched by
// src/flashquant/kernels/attention.py:85-107:
//   q_rot = (q @ R^T) rounded to the query dtype
//   K, V  = centroid[idx] * norm in rotated space
//   out   = (softmax(q_rot K^T * scale + causal mask) V) @ R, rounded once
// The causal mask hides key j > query i counted from the top-left corner and is
// dropped when there is a single query row (cpu_reference.py:97-151).
//
// Work split.  A workgroup of 8 wavefronts serves one (batch, KV head) pair and 8
// "units": a unit is a block of 32 query positions of one query head of the group,
// so with 4 query heads per KV head a workgroup covers 64 positions of all 4 heads
// and every dequantised K/V tile is used for 256 query rows.
//
// Per 64-token tile all 512 threads dequantise K and V into LDS as fp16 with the
// norm folded in (one LDS lookup per packed byte in a byte -> (fp16, fp16) table),
// double buffered, one barrier per tile; then each wavefront runs
//   S^T (64 tokens x 32 rows)  = K_tile . q_rot^T      16 x v_mfma_f32_32x32x16_f16
//   O^T (128 coords x 32 rows) += V_tile^T . P^T        16 x v_mfma_f32_32x32x16_f16
// Both products are transposed so that a lane owns one query row (column l % 32 of
// every accumulator): the running maximum, the denominator and the rescale of O are
// per-lane scalars, and P goes from the S accumulator straight into the B operand
// of the second product.  That works because the contraction index of an MFMA may
// be permuted freely as long as both operands agree: the accumulator registers
// r = 8u .. 8u+7 of lane half hf hold rows 16u + 8a + 4hf + c (e = 4a + c), so the
// V tile stores token 16u + 8a + 4b + c at position 16u + 8b + 4a + c and a lane's
// 8 consecutive positions are exactly its 8 tokens.  The K tile uses the same
// permutation on the coordinates, and the query operand is read to match.
//
// The two head rotations run inside the kernel (prologue and epilogue) on the fp16 MFMA
// with operands split into two fp16 terms, staged through the tile buffers.
#include "fq_common.hpp"
#include "fq_device.hpp"
#include "fq_attention_any_dim.hpp"

namespace fq {

// Tile geometry for head_dim D (64 or 128).
template <int D>
struct PrefillCfg {
    static constexpr int KSTRIDE = 2 * D + 16;            // bytes per token row of the K tile (D fp16 + pad): 4 banks
    static constexpr int KBYTES = 64 * KSTRIDE;           // 17408 at D = 128
    static constexpr int VBYTES = D * 128;                // V^T tile: D coordinate rows x 64 tokens fp16
    static constexpr int BUF = KBYTES + VBYTES;           // 33792 at D = 128
    static constexpr int STAGE = 64 * D;                  // per-wavefront staging area for the rotations
    static constexpr int NKS = D / 16;                    // k-steps of the score product
    static constexpr int NOB = D / 32;                    // 32-coordinate blocks of the output
    static constexpr int NJ = D / 32;                     // 32-wide k-steps of the head rotations
    static constexpr int PB = D / 2;                      // packed bytes per token and head
    // The rotation matrix as MFMA operands (two fp16 terms), shared by the wavefronts of a workgroup:
    // block (column block cb, k-step j) holds one 16-byte operand per lane and term.  They lie where
    // the lookup tables are between the query stage and the end of the tile loop (64 KB).
    static constexpr int RTERM = NKS * NJ * 64 * 16;      // bytes per term: 32768 at D = 128
};

struct PrefillParams {
    const uint16_t* q;          // (B, H_Q, N_Q, 128)
    const uint8_t* k_packed;    // (B, H_KV, N_KV, 64)
    const float* k_norms;       // (B, H_KV, N_KV)
    const uint8_t* v_packed;
    const float* v_norms;
    const float* centroids_k;
    const float* centroids_v;
    const float* rotation;      // (128, 128)
    uint16_t* out;              // (B, H_Q, N_Q, 128)
    int rot_col_major;
    int H_Q, H_KV, G, N_Q, N_KV;
    int64_t k_cap, v_cap;       // tokens between the slabs of consecutive (batch, KV head) pairs (>= N_KV)
    int causal;
    float scale_log2e;
    // paged mode (variable-length queries over the packed paged cache)
    const int32_t* cu_seqlens_q;   // (S + 1,) first query token of every sequence in q / out (tokens, H_Q, 128)
    const int32_t* seq_lens;       // (S,) keys of every sequence, the new tokens included
    const int32_t* block_table;    // (S, max_blocks)
    const uint8_t* cache;          // (num_blocks, block_size, H_KV * 136)
    int max_blocks, num_blocks, bs_log2;
    int round_slots;               // workgroups running at a time (one per CU)
};

__device__ __forceinline__ uint32_t scale_pair(uint32_t pair, half2v n2) {
    const half2v h = __builtin_bit_cast(half2v, pair) * n2;
    return __builtin_bit_cast(uint32_t, h);
}

__device__ __forceinline__ uint32_t pack_rtz(float a, float b) {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(a, b));
}

// PAGED: the sequences' queries are packed along the token axis of q (tokens, H_Q, 128), the keys
// and values come from the paged TQ4 cache through the block table, query j of a sequence with
// n queries and L keys sits at position L - n + j (the new tokens are the last ones), and the
// attention result is rounded to the query dtype before the rotation back, as the attention
// library's output is in the path this replaces (src/flashquant/vllm/impl.py:265-336, 470-512).
template <int D, int DT, bool PAGED>
__global__ __launch_bounds__(512) void fused_tq_attention_kernel(const PrefillParams p) {
    using Cfg = PrefillCfg<D>;
    constexpr int kPfKStride = Cfg::KSTRIDE, kPfKBytes = Cfg::KBYTES, kPfBufBytes = Cfg::BUF, kPfStageBytes = Cfg::STAGE;
    constexpr int NKS = Cfg::NKS, NOB = Cfg::NOB, NJ = Cfg::NJ, PB = Cfg::PB;
    __shared__ __attribute__((aligned(256))) uint32_t lut[256 * 64];
    extern __shared__ __attribute__((aligned(16))) uint8_t bufs[];   // 2 x (K tile | V^T tile)
    // Rows whose norm times a centroid would not fit fp16 are stored divided by a power of two.
    // big_tile[buf] = tile + 1 marks a tile that holds such rows; scale_exp[buf] holds the exponents,
    // K rows 0..63 then V rows 0..63, each tagged with tile + 1 in its upper bits (an entry with
    // another tag is left over from an earlier tile and reads as 0).
    __shared__ int big_tile[2];
    __shared__ __attribute__((aligned(16))) int scale_exp[2][128];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int m32 = lane & 31, hf = lane >> 5;     // 32x32 MFMA: column (query row) and lane half
    const int n16 = lane & 15, g4 = lane >> 4;     // 16x16 MFMA of the rotations
    // Workgroups reach the CUs in the order of their linear index, round after round, and under a
    // causal mask their durations grow with the query position.  Position fastest, (batch, head)
    // slow, and the position order reversed in every other round over the chip: whichever way the
    // rounds land on the CUs, each CU sees long and short workgroups alternate.
    const int lin = int(blockIdx.x) + int(gridDim.x) * (int(blockIdx.y) + int(gridDim.y) * int(blockIdx.z));
    const int pair = lin / int(gridDim.x);
    const int b = pair / int(gridDim.y), hkv = pair % int(gridDim.y);
    const int x_in_pair = lin % int(gridDim.x);
    // The direction is a function of the pair alone (the round its first workgroup falls in), so
    // inside a pair x -> wg is a bijection whatever the grid and the CU count are.
    const bool flip = (((int64_t(pair) * int64_t(gridDim.x)) / p.round_slots) & 1) != 0;

    // ---- this sequence -----------------------------------------------------------------------
    int NQ = p.N_Q, NKV = p.N_KV, qoff = 0;
    int64_t q_row0 = (int64_t(b) * p.H_Q) * p.N_Q;     // first row of head 0 in q / out, in rows of 128
    int q_stride = D;                                  // elements between consecutive positions of a head
    if (PAGED) {
        const int first = p.cu_seqlens_q[b];
        NQ = p.cu_seqlens_q[b + 1] - first;
        NKV = p.seq_lens[b];
        NKV = NKV < 0 ? 0 : (NKV > (p.max_blocks << p.bs_log2) ? (p.max_blocks << p.bs_log2) : NKV);
        qoff = NKV - NQ > 0 ? NKV - NQ : 0;
        q_row0 = int64_t(first) * p.H_Q;
        q_stride = p.H_Q * D;
        if (NQ <= 0) return;
    }

    // ---- units --------------------------------------------------------------------------
    const int nblk = (NQ + 31) >> 5;
    const int units = nblk * p.G;
    const int wg = flip ? x_in_pair : int(gridDim.x) - 1 - x_in_pair;
    if (PAGED && 8 * wg >= units) return;                  // the grid is sized for the longest sequence
    const int unit_raw = 8 * wg + w;
    const bool unit_live = unit_raw < units;
    const int unit = unit_live ? unit_raw : units - 1;
    const int hq = hkv * p.G + unit % p.G;
    const int pos0 = 32 * (unit / p.G);
    const int last_unit = 8 * wg + 7 < units - 1 ? 8 * wg + 7 : units - 1;
    int wg_maxpos = 32 * (last_unit / p.G) + 31;
    wg_maxpos = wg_maxpos < NQ - 1 ? wg_maxpos : NQ - 1;
    int my_maxpos = pos0 + 31 < NQ - 1 ? pos0 + 31 : NQ - 1;
    const int all_tiles = (NKV + 63) >> 6;
    int ntiles = all_tiles, my_tiles = all_tiles;
    if (p.causal) {
        ntiles = ((qoff + wg_maxpos) >> 6) + 1 < all_tiles ? ((qoff + wg_maxpos) >> 6) + 1 : all_tiles;
        my_tiles = ((qoff + my_maxpos) >> 6) + 1 < all_tiles ? ((qoff + my_maxpos) >> 6) + 1 : all_tiles;
    }
    if (!unit_live) my_tiles = 0;

    // ---- tables: filled after the query stage, whose rotation operands use their place ----------
    static_assert(2 * Cfg::RTERM <= int(sizeof(lut)), "the rotation operands fit where the tables are");
    // cleared here: the barriers of the query stage order this before the first dequantisation
    if (tid < 2) big_tile[tid] = 0;
    if (tid < 256) (&scale_exp[0][0])[tid] = 0;
    const uint8_t* lutb = reinterpret_cast<const uint8_t*>(lut);
    const uint32_t lk = 4u * (lane & 31), lv = 128u + lk;

    // ---- dequantisation plan ------------------------------------------------------------------
    const int64_t k_row0 = PAGED ? 0 : (int64_t(b) * p.H_KV + hkv) * p.k_cap;
    const int64_t v_row0 = PAGED ? 0 : (int64_t(b) * p.H_KV + hkv) * p.v_cap;
    const uint8_t* kp = p.k_packed + k_row0 * PB;
    const uint8_t* vp = p.v_packed + v_row0 * PB;
    const float* knp = p.k_norms + k_row0;
    const float* vnp = p.v_norms + v_row0;
    // Work items of the dequantisation.  K: (token of the tile, 16-coordinate group); V: (token pair, dword
    // of the packed row).  head_dim 128: 512 of each, every thread takes one of both; head_dim 64: 256 of
    // each, wavefronts 0..3 take the V items and wavefronts 4..7 the K items.
    constexpr bool kSplitRoles = D == 64;
    const bool does_k = !kSplitRoles || w >= 4;
    const bool does_v = !kSplitRoles || w < 4;
    int gqk, tk, jv, tp;
    if constexpr (!kSplitRoles) {
        // K lane bits (g0 g1 t0 g2 t1 t2): eight consecutive lanes hold four groups of two consecutive
        // tokens, so the 128 bytes they store with one 16-byte write each fall into 32 different banks
        // (token rows are 272 bytes apart: 4 banks).
        gqk = (lane & 3) | ((lane >> 1) & 4);
        tk = 8 * w + ((lane >> 2) & 1) + ((lane >> 3) & 6);
        // V: the four pairs of a wavefront are the ones whose positions share a 16-byte group of the
        // transposed tile (0, 2, 4, 6 within it); lane bits (j0 j1 j2 p0 p1 j3): each half of the
        // wavefront holds all four pairs and eight dwords, so that its store covers all 32 banks once.
        jv = (lane & 7) | ((lane >> 2) & 8);
        tp = 8 * (w >> 1) + 2 * (w & 1) + ((lane >> 3) & 1) + 4 * ((lane >> 4) & 1);
    } else {
        // K (wavefronts 4..7): lane bits (g0 g1 t0 t1 t2 t3), 16 tokens per wavefront
        gqk = lane & 3;
        tk = 16 * (w & 3) + (lane >> 2);
        // V (wavefronts 0..3): lane bits (j0 j1 j2 p0 p1 p2): eight pairs per wavefront, the four of
        // each half sharing a 16-byte group of the transposed tile
        jv = lane & 7;
        const int i8 = lane >> 3;                       // 0..7
        tp = 8 * (w & 3) + 2 * (i8 >> 2) + (i8 & 1) + 4 * ((i8 >> 1) & 1);
    }
    const int k_wr = tk * kPfKStride + gqk * 32;
    int v_wr[8];
    {
        const int tt = 2 * tp, t16 = tt & 15;
        const int posv = (tt & ~15) + 8 * ((t16 >> 2) & 1) + 4 * ((t16 >> 3) & 1) + (t16 & 3);
        const int giv = posv >> 3, within = posv & 7;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int d = 8 * jv + k;
            const int physg = giv ^ k ^ (jv & 7);
            v_wr[k] = kPfKBytes + d * 128 + 16 * physg + 2 * within;
        }
    }
    uint2v kraw = {0u, 0u};
    uint32_t vra = 0u, vrb = 0u;
    float nk = 0.0f, nv0 = 0.0f, nv1 = 0.0f;
    auto issue_loads = [&](int tile_raw) {
        const int tile = tile_raw < ntiles ? tile_raw : ntiles - 1;   // past the end: the last tile again, never used
        const int t0 = tile > 0 ? tile * 64 : 0;
        const int last = NKV > 0 ? NKV - 1 : 0;
        const int tkk = t0 + tk < last ? t0 + tk : last;
        const int ta = t0 + 2 * tp < last ? t0 + 2 * tp : last;
        const int tb = t0 + 2 * tp + 1 < last ? t0 + 2 * tp + 1 : last;
        if (PAGED) {
            // token t of the sequence: row t % BS of page block_table[t / BS]; the row holds
            // [K idx H*64 | K norm H*4 | V idx H*64 | V norm H*4]
            const int H = p.H_KV;
            const int64_t row_bytes = int64_t(H) * (D + 8);
            const int32_t* bt = p.block_table + int64_t(b) * p.max_blocks;
            auto row_ptr = [&](int t) {
                int pg = bt[t >> p.bs_log2];
                pg = pg < 0 ? 0 : (pg >= p.num_blocks ? p.num_blocks - 1 : pg);
                return p.cache + ((int64_t(pg) << p.bs_log2) + (t & ((1 << p.bs_log2) - 1))) * row_bytes;
            };
            if (does_k) {
                const uint8_t* rk = row_ptr(tkk);
                kraw = *reinterpret_cast<const uint2v*>(rk + hkv * PB + 8 * gqk);
                nk = *reinterpret_cast<const float*>(rk + H * PB + 4 * hkv);
            }
            if (does_v) {
                const uint8_t* ra = row_ptr(ta);
                const uint8_t* rb2 = row_ptr(tb);
                vra = *reinterpret_cast<const uint32_t*>(ra + H * (PB + 4) + hkv * PB + 4 * jv);
                vrb = *reinterpret_cast<const uint32_t*>(rb2 + H * (PB + 4) + hkv * PB + 4 * jv);
                nv0 = *reinterpret_cast<const float*>(ra + H * (D + 4) + 4 * hkv);
                nv1 = *reinterpret_cast<const float*>(rb2 + H * (D + 4) + 4 * hkv);
            }
        } else {
            // (32-bit offsets from the wave-uniform slab pointers: a slab of 2^31 / PB tokens is far beyond
            // any context)
            if (does_k) {
                kraw = *reinterpret_cast<const uint2v*>(kp + (uint32_t(tkk) * uint32_t(PB) + 8u * uint32_t(gqk)));
                nk = knp[uint32_t(tkk)];
            }
            if (does_v) {
                vra = *reinterpret_cast<const uint32_t*>(vp + (uint32_t(ta) * uint32_t(PB) + 4u * uint32_t(jv)));
                vrb = *reinterpret_cast<const uint32_t*>(vp + (uint32_t(tb) * uint32_t(PB) + 4u * uint32_t(jv)));
                nv0 = vnp[uint32_t(ta)];
                nv1 = vnp[uint32_t(tb)];
            }
        }
    };
    auto dequant = [&](int buf, int tile) {
        uint8_t* dst = bufs + buf * kPfBufBytes;
        if (__any(__builtin_fmaxf(__builtin_fabsf(nk), __builtin_fmaxf(__builtin_fabsf(nv0), __builtin_fabsf(nv1))) >= 32768.0f)) {
            const int ek = norm_excess(nk), ev0 = norm_excess(nv0), ev1 = norm_excess(nv1);
            nk = __builtin_ldexpf(nk, -ek);
            nv0 = __builtin_ldexpf(nv0, -ev0);
            nv1 = __builtin_ldexpf(nv1, -ev1);
            const int tag = (tile + 1) << 8;
            if (does_k && gqk == 0) scale_exp[buf][tk] = tag | ek;
            if (does_v && jv == 0) {
                scale_exp[buf][64 + 2 * tp] = tag | ev0;
                scale_exp[buf][64 + 2 * tp + 1] = tag | ev1;
            }
            if ((ek | ev0 | ev1) != 0) big_tile[buf] = tile + 1;
        }
        if (does_k) {      // uniform over the wavefront
            const _Float16 hk = _Float16(nk);
            const half2v nk2 = {hk, hk};
            const uint4v a0 = lookup_word(lutb, kraw.x, lk);   // coordinates 0..7 of the group
            const uint4v a1 = lookup_word(lutb, kraw.y, lk);   // coordinates 8..15
            // positions 0..7 = coordinates (0..3, 8..11), positions 8..15 = (4..7, 12..15)
            const uint4v w0 = {scale_pair(a0.x, nk2), scale_pair(a0.y, nk2), scale_pair(a1.x, nk2), scale_pair(a1.y, nk2)};
            const uint4v w1 = {scale_pair(a0.z, nk2), scale_pair(a0.w, nk2), scale_pair(a1.z, nk2), scale_pair(a1.w, nk2)};
            *reinterpret_cast<uint4v*>(dst + k_wr) = w0;
            *reinterpret_cast<uint4v*>(dst + k_wr + 16) = w1;
        }
        if (does_v) {
            // V: 2x2 nibble transpose, so that a byte holds one coordinate of the two tokens
            const uint32_t X = (vra & 0xF0F0F0F0u) | ((vrb >> 4) & 0x0F0F0F0Fu);   // even coordinates
            const uint32_t Y = ((vra << 4) & 0xF0F0F0F0u) | (vrb & 0x0F0F0F0Fu);   // odd coordinates
            const half2v nv2 = {_Float16(nv0), _Float16(nv1)};
            const uint4v xe = lookup_word(lutb, X, lv);
            const uint4v yo = lookup_word(lutb, Y, lv);
            const uint32_t xs[4] = {xe.x, xe.y, xe.z, xe.w}, ys[4] = {yo.x, yo.y, yo.z, yo.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                *reinterpret_cast<uint32_t*>(dst + v_wr[2 * c]) = scale_pair(xs[c], nv2);
                *reinterpret_cast<uint32_t*>(dst + v_wr[2 * c + 1]) = scale_pair(ys[c], nv2);
            }
        }
    };

    issue_loads(0);

    // ---- the rotation matrix, split once per workgroup ------------------------------------------------
    // Wavefront cb fetches column block cb of R^T (or of R), splits it into two fp16 terms and
    // leaves the operands in LDS; every wavefront then reads the blocks it multiplies with from
    // there (each wavefront fetching and splitting the whole matrix for itself, three times per
    // workgroup, was an eighth of the kernel's time).
    uint8_t* rshare = reinterpret_cast<uint8_t*>(lut);
    auto share_rotation = [&](bool transposed) {
        if (w < NKS) {
            float rbv[NJ][8];
            load_rotation_any<D>(p.rotation, p.rot_col_major != 0, transposed, 16 * w, n16, g4, rbv);
            half8 rhi[NJ], rlo[NJ];
            split_rotation_block<D>(rbv, rhi, rlo);
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                *reinterpret_cast<half8*>(rshare + ((w * NJ + j) * 64 + lane) * 16) = rhi[j];
                *reinterpret_cast<half8*>(rshare + Cfg::RTERM + ((w * NJ + j) * 64 + lane) * 16) = rlo[j];
            }
        }
    };
    auto shared_rotation_block = [&](int cb, half8 (&rhi)[NJ], half8 (&rlo)[NJ]) {
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            rhi[j] = *reinterpret_cast<const half8*>(rshare + ((cb * NJ + j) * 64 + lane) * 16);
            rlo[j] = *reinterpret_cast<const half8*>(rshare + Cfg::RTERM + ((cb * NJ + j) * 64 + lane) * 16);
        }
    };

    // ---- query: rotate this wavefront's 32 rows, round to the query dtype, scale to fp16 ----------
    half8 qb[NKS];
    float krow;
    {
        const uint16_t* qbase = PAGED ? p.q + (q_row0 + hq) * D : p.q + (q_row0 + int64_t(hq) * NQ) * D;
        uint16_t* st = reinterpret_cast<uint16_t*>(bufs + w * kPfStageBytes);   // (32 rows, D) raw 16-bit
        // the rows are exact in fp16 up to a power of two: fp16-split MFMA, two terms
        half8 a[2][NJ];
        float up[2];
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            int pos = pos0 + 16 * rb + n16;
            pos = pos < NQ ? pos : NQ - 1;
            uint4v raw[NJ];
#pragma unroll
            for (int j = 0; j < NJ; ++j) raw[j] = *reinterpret_cast<const uint4v*>(qbase + int64_t(pos) * q_stride + 32 * j + 8 * g4);
            rows_as_f16<D, DT>(raw, a[rb], up[rb]);
        }
        share_rotation(true);
        __syncthreads();
        for (int cb = 0; cb < NKS; ++cb) {
            half8 rhi[NJ], rlo[NJ];
            shared_rotation_block(cb, rhi, rlo);
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                const float4v acc = rotate_block_f16<D>(a[rb], rhi, rlo);
#pragma unroll
                for (int i = 0; i < 4; ++i) st[(16 * rb + 4 * g4 + i) * D + 16 * cb + n16] = store_elem<DT>(acc[i] * up[rb]);
            }
        }
        __syncthreads();
        float qf[NKS][8];
        float mx = 0.0f;
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
            const uint2v lo = *reinterpret_cast<const uint2v*>(st + m32 * D + 16 * ks + 4 * hf);
            const uint2v hi = *reinterpret_cast<const uint2v*>(st + m32 * D + 16 * ks + 8 + 4 * hf);
            const uint32_t wds[4] = {lo.x, lo.y, hi.x, hi.y};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                qf[ks][2 * i] = load_elem<DT>(uint16_t(wds[i] & 0xffffu));
                qf[ks][2 * i + 1] = load_elem<DT>(uint16_t(wds[i] >> 16));
                mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(qf[ks][2 * i]), __builtin_fabsf(qf[ks][2 * i + 1])));
            }
        }
        mx = __builtin_fmaxf(mx, xor_shuffle(mx, 32));
        int ex = int((float_to_bits(mx) >> 23) & 0xffu) - 127;
        if (ex < -100 || ex > 100) ex = 0;
        const float down = bits_to_float(uint32_t(127 - ex) << 23);
        krow = p.scale_log2e * bits_to_float(uint32_t(127 + ex) << 23);
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) qb[ks][e] = _Float16(qf[ks][e] * down);
        __syncthreads();   // the staging area becomes tile buffers, the rotation operands lookup tables
    }
    fill_pair_tables<8>(lut, p.centroids_k[lane & 15], p.centroids_v[lane & 15], 15, w, lane);
    __syncthreads();

    // ---- lane-constant LDS read offsets ----------------------------------------------------------
    const int k_rd = m32 * kPfKStride + 16 * hf;
    int v_rd[8];
    {
        const int lanex = hf ^ (m32 & 7) ^ (m32 >> 3);
#pragma unroll
        for (int c = 0; c < 8; ++c) v_rd[c] = kPfKBytes + m32 * 128 + 16 * (lanex ^ c);
    }

    // ---- running state -----------------------------------------------------------------------------
    float16v O[NOB];
#pragma unroll
    for (int ob = 0; ob < NOB; ++ob)
#pragma unroll
        for (int r = 0; r < 16; ++r) O[ob][r] = 0.0f;
    float m_run = -__builtin_inff();
    float l_run = 0.0f;
    const int qpos = qoff + pos0 + m32;            // position among the keys

    auto compute = [&](int tile, int buf) {
        const uint8_t* kt = bufs + buf * kPfBufBytes;
        float16v S[2];
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) S[tb][r] = 0.0f;
#pragma unroll
            for (int ks = 0; ks < NKS; ++ks) {
                const half8 a = *reinterpret_cast<const half8*>(kt + k_rd + 32 * tb * kPfKStride + 32 * ks);
                S[tb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qb[ks], S[tb], 0, 0, 0);
            }
        }
        const int t0 = tile * 64;
        // rows stored divided by a power of two (norms beyond fp16's range): wavefront-uniform, rare
        const bool big = __builtin_amdgcn_readfirstlane(big_tile[buf]) == tile + 1;
        auto exps_of = [&](int first) {        // the exponents of four consecutive rows of this tile
            const int4v raw = *reinterpret_cast<const int4v*>(&scale_exp[buf][first]);
            int4v e;
#pragma unroll
            for (int c = 0; c < 4; ++c) e[c] = (raw[c] >> 8) == tile + 1 ? (raw[c] & 0xff) : 0;
            return e;
        };
        if (big) {
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int4v e = exps_of(32 * tb + 8 * q + 4 * hf);
#pragma unroll
                    for (int c = 0; c < 4; ++c) S[tb][4 * q + c] = __builtin_ldexpf(S[tb][4 * q + c], e[c]);
                }
        }
        const bool need_mask = (t0 + 63 >= NKV) || (p.causal && t0 + 63 > qoff + pos0);   // wavefront-uniform
        if (need_mask) {
            int lim = NKV - 1;
            if (p.causal && qpos < lim) lim = qpos;
            lim -= t0;                         // token offsets <= lim are visible
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int off = 32 * tb + 8 * (r >> 2) + 4 * hf + (r & 3);
                    if (off > lim) S[tb][r] = -__builtin_inff();
                }
        }
        float cand;
        if (!big) {
            float mx = S[0][0];
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = __builtin_fmaxf(mx, S[tb][r]);
            cand = mx * krow;
        } else {
            // a value row stored divided by 2^e gets its weight multiplied by 2^e: the reference is
            // taken over score + e, so that these weights stay below 16 as well
            cand = -__builtin_inff();
#pragma unroll
            for (int tb = 0; tb < 2; ++tb)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int4v e = exps_of(64 + 32 * tb + 8 * q + 4 * hf);
#pragma unroll
                    for (int c = 0; c < 4; ++c)
                        cand = __builtin_fmaxf(cand, __builtin_fmaf(S[tb][4 * q + c], krow, float(e[c])));
                }
        }
        cand = max_xor32(cand);
        // the running maximum moves only when it would grow by more than 2^4: the weights stay
        // below 16 and the rescale of the accumulator registers becomes rare
        const float mnew = cand > m_run + 4.0f ? cand : m_run;
        const float ms = mnew == -__builtin_inff() ? 0.0f : mnew;
        const float alpha = __builtin_amdgcn_exp2f(m_run - ms);
        m_run = mnew;
        uint4v pbv[4];
        float ps = 0.0f;
        // two copies of the weight loop, so that the common one has no branch inside (the values of a
        // loop with a rare branch in it are copied where the paths meet)
        if (!big) {
            const half2v ones = {_Float16(1.0f), _Float16(1.0f)};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                float pe[8];
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    pe[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(S[s >> 1][8 * (s & 1) + e], krow, -ms));
                const uint32_t pw[4] = {pack_rtz(pe[0], pe[1]), pack_rtz(pe[2], pe[3]), pack_rtz(pe[4], pe[5]), pack_rtz(pe[6], pe[7])};
                // the denominator sums the weights as the second product sees them (fp16, one
                // v_dot2_f32_f16 per pair)
#pragma unroll
                for (int c = 0; c < 4; ++c) ps = __builtin_amdgcn_fdot2(__builtin_bit_cast(half2v, pw[c]), ones, ps, false);
                pbv[s] = uint4v{pw[0], pw[1], pw[2], pw[3]};
            }
        } else {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                float pe[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    pe[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(S[s >> 1][8 * (s & 1) + e], krow, -ms));
                    ps += pe[e];
                }
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    const int4v ev = exps_of(64 + 32 * (s >> 1) + 8 * (2 * (s & 1) + q) + 4 * hf);
#pragma unroll
                    for (int c = 0; c < 4; ++c) pe[4 * q + c] = __builtin_ldexpf(pe[4 * q + c], ev[c]);
                }
                pbv[s] = uint4v{pack_rtz(pe[0], pe[1]), pack_rtz(pe[2], pe[3]), pack_rtz(pe[4], pe[5]), pack_rtz(pe[6], pe[7])};
            }
        }
        l_run = __builtin_fmaf(l_run, alpha, ps);
        if (__any(alpha != 1.0f)) {
#pragma unroll
            for (int ob = 0; ob < NOB; ++ob)
#pragma unroll
                for (int r = 0; r < 16; ++r) O[ob][r] *= alpha;
        }
        // The V operands of 16 tokens (one per 32-coordinate block) are read two such groups ahead of
        // the products that use them (the compiler on its own reads one product ahead, which does
        // not cover the LDS round trip): fences keep the groups in this order.
        auto v_operand = [&](int ob, int s) {
            const int c = (2 * s) ^ (4 * (ob & 1));
            return *reinterpret_cast<const half8*>(kt + v_rd[c] + ob * 4096);
        };
        half8 va[4][NOB];
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int ob = 0; ob < NOB; ++ob) va[s][ob] = v_operand(ob, s);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            if (s + 2 < 4) {
#pragma unroll
                for (int ob = 0; ob < NOB; ++ob) va[s + 2][ob] = v_operand(ob, s + 2);
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (int ob = 0; ob < NOB; ++ob)
                O[ob] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[s][ob], __builtin_bit_cast(half8, pbv[s]), O[ob], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- tiles ----------------------------------------------------------------------------------------
    dequant(0, 0);
    issue_loads(1);
    // The dequantisation of tile i + 1 and the products of tile i sit in one basic block (no
    // conditions between them), so that the lookups and LDS writes of the one interleave with
    // the MFMAs of the other.
    int i = 0;
    for (; i < my_tiles; ++i) {
        __syncthreads();                       // tile i is complete; the other buffer is free
        dequant((i + 1) & 1, i + 1);
        issue_loads(i + 2);
        compute(i, i & 1);
    }
    for (; i < ntiles; ++i) {                  // tiles only the other wavefronts of the workgroup need
        __syncthreads();
        dequant((i + 1) & 1, i + 1);
        issue_loads(i + 2);
    }

    // ---- normalise, rotate back, store -------------------------------------------------------------------
    const float l_tot = l_run + xor_shuffle(l_run, 32);
    const float inv = l_tot > 0.0f ? 1.0f / l_tot : 0.0f;
    float* stf = reinterpret_cast<float*>(bufs + w * kPfStageBytes);   // (16 rows, D) float32
    uint16_t* obase = PAGED ? p.out + (q_row0 + hq) * D : p.out + (q_row0 + int64_t(hq) * NQ) * D;
    __syncthreads();                // every wavefront is done with the lookup tables
    share_rotation(false);          // (the barrier below orders it before its readers)
    for (int half_rows = 0; half_rows < 2; ++half_rows) {
        __syncthreads();
        if ((m32 >> 4) == half_rows) {
#pragma unroll
            for (int ob = 0; ob < NOB; ++ob)
#pragma unroll
                for (int rq = 0; rq < 4; ++rq) {
                    float4v v = {O[ob][4 * rq] * inv, O[ob][4 * rq + 1] * inv, O[ob][4 * rq + 2] * inv, O[ob][4 * rq + 3] * inv};
                    if (PAGED) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = load_elem<DT>(store_elem<DT>(v[e]));
                    }
                    *reinterpret_cast<float4v*>(stf + (m32 & 15) * D + 32 * ob + 8 * rq + 4 * hf) = v;
                }
        }
        __syncthreads();
        float a[NJ][8];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
            const float4v lo = *reinterpret_cast<const float4v*>(stf + n16 * D + 32 * j + 8 * g4);
            const float4v hi = *reinterpret_cast<const float4v*>(stf + n16 * D + 32 * j + 8 * g4 + 4);
            a[j][0] = lo.x; a[j][1] = lo.y; a[j][2] = lo.z; a[j][3] = lo.w;
            a[j][4] = hi.x; a[j][5] = hi.y; a[j][6] = hi.z; a[j][7] = hi.w;
        }
        // float32 rows: both operands as two fp16 terms, three MFMA terms
        half8 ahi[NJ], alo[NJ];
        float up;
        rows_split_f16<D>(a, ahi, alo, up);
        for (int cb = 0; cb < NKS; ++cb) {
            half8 rhi[NJ], rlo[NJ];
            shared_rotation_block(cb, rhi, rlo);
            const float4v acc = rotate_block_f16x3<D>(ahi, alo, rhi, rlo);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int pos = pos0 + 16 * half_rows + 4 * g4 + i;
                if (unit_live && pos < NQ) obase[int64_t(pos) * q_stride + 16 * cb + n16] = store_elem<DT>(acc[i] * up);
            }
        }
    }
}

template <int D, bool PAGED>
int launch_prefill(const PrefillParams& p, dim3 grid, int dtype, hipStream_t s) {
    const size_t lds = 2 * size_t(PrefillCfg<D>::BUF);
    const dim3 block(512);
    if (dtype == FQ_F16) {
        auto kern = fused_tq_attention_kernel<D, FQ_F16, PAGED>;
        if (!fq_host::lds_limit_raised(reinterpret_cast<const void*>(kern), lds)) return FQ_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, block, lds, s, p);
    } else {
        auto kern = fused_tq_attention_kernel<D, FQ_BF16, PAGED>;
        if (!fq_host::lds_limit_raised(reinterpret_cast<const void*>(kern), lds)) return FQ_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, block, lds, s, p);
    }
    return fq_host::check_launch();
}

}  // namespace fq

extern "C" int fq_fused_tq_attention(const void* q, const uint8_t* k_packed, const float* k_norms,
                                     const uint8_t* v_packed, const float* v_norms,
                                     const float* centroids_k, const float* centroids_v,
                                     const float* rotation, int rotation_col_major, void* out,
                                     int B, int H_Q, int H_KV, int N_Q, int N_KV, int D,
                                     float sm_scale, int is_causal, int dtype, void* stream) {
    return fq_fused_tq_attention_strided(q, k_packed, k_norms, v_packed, v_norms, centroids_k, centroids_v, rotation,
                                         rotation_col_major, out, B, H_Q, H_KV, N_Q, N_KV, N_KV, N_KV, D, sm_scale,
                                         is_causal, dtype, stream);
}

extern "C" int fq_fused_tq_attention_strided(const void* q, const uint8_t* k_packed, const float* k_norms,
                                             const uint8_t* v_packed, const float* v_norms,
                                             const float* centroids_k, const float* centroids_v,
                                             const float* rotation, int rotation_col_major, void* out,
                                             int B, int H_Q, int H_KV, int N_Q, int N_KV,
                                             int64_t k_capacity, int64_t v_capacity, int D,
                                             float sm_scale, int is_causal, int dtype, void* stream) {
    using namespace fq;
    if (B < 0 || H_Q <= 0 || H_KV <= 0 || N_Q < 0 || N_KV < 0 || H_Q % H_KV != 0) return FQ_ERR_BAD_SHAPE;
    if (k_capacity < N_KV || v_capacity < N_KV) return FQ_ERR_BAD_SHAPE;
    if (N_KV > (1 << 24)) return FQ_ERR_BAD_SHAPE;      // the kernels address a slab's tokens with 32-bit byte offsets
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (dtype != FQ_F16 && dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (B == 0 || N_Q == 0) return FQ_OK;
    if (N_KV == 0) return FQ_ERR_BAD_SHAPE;          // softmax over no keys is undefined
    if (!q || !k_packed || !k_norms || !v_packed || !v_norms || !centroids_k || !centroids_v || !rotation || !out)
        return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(q, 16) || !fq_host::aligned(k_packed, 8) || !fq_host::aligned(v_packed, 4) ||
        !fq_host::aligned(rotation, 16) || !fq_host::aligned(out, 2))
        return FQ_ERR_MISALIGNED;
    if (B > 65535 || H_KV > 65535) return FQ_ERR_BAD_SHAPE;

    if (D == 256 || fq_host::force_any_dim_attention()) {   // the tuned tile layout serves 64 and 128 coordinates
        AnyDimParams a{};
        a.q = static_cast<const uint16_t*>(q);
        a.k_packed = k_packed; a.k_norms = k_norms; a.v_packed = v_packed; a.v_norms = v_norms;
        a.centroids_k = centroids_k; a.centroids_v = centroids_v;
        a.rotation = rotation; a.rot_col_major = rotation_col_major;
        a.out = static_cast<uint16_t*>(out);
        a.H_Q = H_Q; a.H_KV = H_KV; a.G = H_Q / H_KV; a.N_Q = N_Q; a.N_KV = N_KV;
        a.k_cap = k_capacity; a.v_cap = v_capacity;
        a.causal = (is_causal && N_Q > 1) ? 1 : 0;
        a.scale_log2e = sm_scale * kLog2e;
        return launch_attention_any_dim(a, D, false, N_Q, B, dtype, stream);
    }

    PrefillParams p;
    p.q = static_cast<const uint16_t*>(q);
    p.k_packed = k_packed; p.k_norms = k_norms; p.v_packed = v_packed; p.v_norms = v_norms;
    p.centroids_k = centroids_k; p.centroids_v = centroids_v;
    p.rotation = rotation; p.rot_col_major = rotation_col_major;
    p.out = static_cast<uint16_t*>(out);
    p.H_Q = H_Q; p.H_KV = H_KV; p.G = H_Q / H_KV; p.N_Q = N_Q; p.N_KV = N_KV;
    p.k_cap = k_capacity; p.v_cap = v_capacity;
    p.causal = (is_causal && N_Q > 1) ? 1 : 0;
    p.scale_log2e = sm_scale * kLog2e;

    const int64_t units = int64_t((N_Q + 31) / 32) * p.G;
    const int64_t wgs = (units + 7) / 8;
    if (wgs > 0x7fffffffLL) return FQ_ERR_BAD_SHAPE;
    const dim3 grid(static_cast<unsigned>(wgs), H_KV, B);
    hipStream_t s = static_cast<hipStream_t>(stream);
    p.cu_seqlens_q = nullptr; p.seq_lens = nullptr; p.block_table = nullptr; p.cache = nullptr;
    p.max_blocks = 0; p.num_blocks = 0; p.bs_log2 = 0;
    p.round_slots = fq_host::device_cu_count();
    return D == 64 ? launch_prefill<64, false>(p, grid, dtype, s) : launch_prefill<128, false>(p, grid, dtype, s);
}

extern "C" int fq_paged_tq4_prefill(const void* q, const int32_t* cu_seqlens_q, const uint8_t* kv_cache,
                                    const int32_t* block_table, const int32_t* seq_lens,
                                    const float* centroids_k, const float* centroids_v,
                                    const float* rotation, int rotation_col_major, void* out,
                                    int num_seqs, int max_q_len, int H_Q, int H_KV, int D, int block_size,
                                    int max_blocks_per_seq, int64_t num_blocks, float sm_scale, int is_causal,
                                    int dtype, void* stream) {
    using namespace fq;
    if (num_seqs < 0 || max_q_len < 0 || H_Q <= 0 || H_KV <= 0 || H_Q % H_KV != 0 || max_blocks_per_seq <= 0 ||
        num_blocks <= 0 || num_blocks > 0x7fffffffLL)
        return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (block_size != 8 && block_size != 16 && block_size != 32) return FQ_ERR_UNSUPPORTED_BLOCK;
    if (dtype != FQ_F16 && dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (num_seqs == 0 || max_q_len == 0) return FQ_OK;
    if (!q || !cu_seqlens_q || !kv_cache || !block_table || !seq_lens || !centroids_k || !centroids_v || !rotation || !out)
        return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(q, 16) || !fq_host::aligned(kv_cache, 16) || !fq_host::aligned(rotation, 16) ||
        !fq_host::aligned(out, 2))
        return FQ_ERR_MISALIGNED;
    if (num_seqs > 65535 || H_KV > 65535) return FQ_ERR_BAD_SHAPE;

    if (D == 256 || fq_host::force_any_dim_attention()) {
        AnyDimParams a{};
        a.q = static_cast<const uint16_t*>(q);
        a.centroids_k = centroids_k; a.centroids_v = centroids_v;
        a.rotation = rotation; a.rot_col_major = rotation_col_major;
        a.out = static_cast<uint16_t*>(out);
        a.H_Q = H_Q; a.H_KV = H_KV; a.G = H_Q / H_KV;
        a.causal = is_causal ? 1 : 0;
        a.scale_log2e = sm_scale * kLog2e;
        a.cu_seqlens_q = cu_seqlens_q; a.seq_lens = seq_lens; a.block_table = block_table; a.cache = kv_cache;
        a.max_blocks = max_blocks_per_seq; a.num_blocks = int(num_blocks);
        a.bs_log2 = block_size == 8 ? 3 : (block_size == 16 ? 4 : 5);
        return launch_attention_any_dim(a, D, true, max_q_len, num_seqs, dtype, stream);
    }

    PrefillParams p;
    p.q = static_cast<const uint16_t*>(q);
    p.k_packed = nullptr; p.k_norms = nullptr; p.v_packed = nullptr; p.v_norms = nullptr;
    p.centroids_k = centroids_k; p.centroids_v = centroids_v;
    p.rotation = rotation; p.rot_col_major = rotation_col_major;
    p.out = static_cast<uint16_t*>(out);
    p.H_Q = H_Q; p.H_KV = H_KV; p.G = H_Q / H_KV; p.N_Q = 0; p.N_KV = 0;
    p.k_cap = 0; p.v_cap = 0;
    p.causal = is_causal ? 1 : 0;
    p.scale_log2e = sm_scale * kLog2e;
    p.cu_seqlens_q = cu_seqlens_q; p.seq_lens = seq_lens; p.block_table = block_table; p.cache = kv_cache;
    p.max_blocks = max_blocks_per_seq; p.num_blocks = int(num_blocks);
    p.bs_log2 = block_size == 8 ? 3 : (block_size == 16 ? 4 : 5);
    p.round_slots = fq_host::device_cu_count();

    const int64_t units = int64_t((max_q_len + 31) / 32) * p.G;
    const int64_t wgs = (units + 7) / 8;
    if (wgs > 0x7fffffffLL) return FQ_ERR_BAD_SHAPE;
    const dim3 grid(static_cast<unsigned>(wgs), H_KV, num_seqs);
    hipStream_t s = static_cast<hipStream_t>(stream);
    return D == 64 ? launch_prefill<64, true>(p, grid, dtype, s) : launch_prefill<128, true>(p, grid, dtype, s);
}
