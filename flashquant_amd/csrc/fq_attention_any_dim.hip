// Fused TQ4 attention for head_dim 64 and 256 (and, as a cross-check, 128): the operator of
// fq_fused_attention.hip (src/flashquant/kernels/cpu_reference.py:154-227, the launcher
// csrc/cuda/fused_tq_attention.cu:468-511 takes all three dimensions) in a plainer shape.
// The tuned kernel's tile layout is written for 128 coordinates; this one trades speed for
// generality and shares nothing with it but the arithmetic rules:
//   q_rot = (q @ R^T) rounded to the query dtype (float32 MFMA)
//   K, V  = fp16(centroid[idx] * norm), scores and P.V on v_mfma_f32_16x16x32_f16
//   out   = (softmax(...) V) @ R, rounded once (contiguous operands) or rounded before and after
//           the rotation (paged operands, as the serving path rounds)
//
// A workgroup of 8 wavefronts owns 128 query rows that share their keys and values, 16 per wavefront:
// 64 positions of two query heads of one KV head (an even number of query heads per KV head), else 128
// positions of one query head.  One workgroup per CU: its byte -> centroid-pair tables are kept in 32
// copies (one per bank, as in the decode kernels), and a tile is dequantised once for 128 rows.  Per
// 32-token tile all threads dequantise K (row-major) and V (transposed) into LDS; a wavefront
// then computes S = q K^T in the MFMA accumulator layout (lane = token column, registers = 4 query
// rows), keeps the running maximum per row with row-wide DPP reductions, moves P through a
// private LDS patch into the A-operand layout, and accumulates O (registers = the same 4 rows,
// so the rescale needs no cross-lane traffic).
#include <cstdlib>

#include "fq_common.hpp"
#include "fq_device.hpp"
#include "fq_attention_any_dim.hpp"

namespace fq {


// maximum over the 16 lanes of a DPP row
__device__ __forceinline__ float row16_max(float v) {
    v = __builtin_fmaxf(v, dpp_mov<0x121>(v));
    v = __builtin_fmaxf(v, dpp_mov<0x122>(v));
    v = __builtin_fmaxf(v, dpp_mov<0x124>(v));
    v = __builtin_fmaxf(v, dpp_mov<0x128>(v));
    return v;
}
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_mov<0x121>(v);
    v += dpp_mov<0x122>(v);
    v += dpp_mov<0x124>(v);
    v += dpp_mov<0x128>(v);
    return v;
}

template <int D>
struct AnyDimCfg {
    static constexpr int KSTRIDE = D + 8;                 // halves per K tile row (padded)
    static constexpr int VSTRIDE = 32 + 8;                // halves per V^T tile row
    static constexpr int K_BYTES = 32 * KSTRIDE * 2;
    static constexpr int V_BYTES = D * VSTRIDE * 2;
    static constexpr int WAVES = 8;
    static constexpr int P_BYTES = WAVES * 16 * VSTRIDE * 2;  // one 16 x 32 patch per wavefront
    static constexpr int Q_BYTES = WAVES * 16 * KSTRIDE * 2;  // rotated query rows, fp16: before the loop, over the tiles
    static constexpr int LOOP_BYTES = K_BYTES + V_BYTES + P_BYTES;
    static constexpr int O_BYTES = 4 * 16 * (D + 4) * 4;  // float32 rows for the rotation back, four wavefronts at a time
    static constexpr int LDS_BYTES = (LOOP_BYTES > O_BYTES ? LOOP_BYTES : O_BYTES) > Q_BYTES
                                         ? (LOOP_BYTES > O_BYTES ? LOOP_BYTES : O_BYTES) : Q_BYTES;
    static constexpr int COPIES = 32;                     // of each byte -> centroid-pair table
};

template <int D, int DT, bool PAGED>
__global__ __launch_bounds__(512) void tq_attention_any_dim_kernel(const AnyDimParams p) {
    using C = AnyDimCfg<D>;
    constexpr int NJ = D / 32;          // k-steps of the score product
    constexpr int NCB = D / 16;         // 16-coordinate output blocks
    constexpr int BPT = D / 64;         // packed bytes per thread and token in the dequantisation (32 threads per token pair)
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    // byte -> (fp16 centroid[high nibble], fp16 centroid[low nibble]); for V the two nibbles of the byte
    // come from two consecutive tokens (see the dequantisation)
    // (entry b of copy c at word 32 b + c: a half-wave's lookups never share a bank)
    __shared__ __attribute__((aligned(16))) uint32_t pair_k[256 * C::COPIES], pair_v[256 * C::COPIES];
    // A row whose norm lies above 2^15 is stored divided by 2^excess (its products with a centroid
    // then fit fp16); the power of two goes back in on the float32 score (K) or weight (V).
    __shared__ int k_exc[32], v_exc[32];
    _Float16* ks = reinterpret_cast<_Float16*>(smem);
    _Float16* vt = reinterpret_cast<_Float16*>(smem + C::K_BYTES);
    _Float16* ps = reinterpret_cast<_Float16*>(smem + C::K_BYTES + C::V_BYTES);
    _Float16* qs = reinterpret_cast<_Float16*>(smem);      // before the first tile is dequantised

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int w = tid >> 6;
    const int wl = w & 3, wg = w >> 2;                // wavefront of its group of four, group
    const int n16 = lane & 15, g4 = lane >> 4;
    const int copy = lane & 31;
    // the two groups: two query heads of one KV head on the same 64 positions, or one head on 128 positions
    const bool two_heads = (p.G & 1) == 0;
    const int hq = two_heads ? 2 * int(blockIdx.y) + wg : int(blockIdx.y), b = blockIdx.z;
    const int hkv = hq / p.G;

    int NQ = p.N_Q, NKV = p.N_KV, qoff = 0;
    int64_t q_row0 = (int64_t(b) * p.H_Q + hq) * p.N_Q;   // first row of this head, in rows of D
    int q_stride = D;
    if (PAGED) {
        const int first = p.cu_seqlens_q[b];
        NQ = p.cu_seqlens_q[b + 1] - first;
        NKV = p.seq_lens[b];
        NKV = NKV < 0 ? 0 : (NKV > (p.max_blocks << p.bs_log2) ? (p.max_blocks << p.bs_log2) : NKV);
        qoff = NKV - NQ > 0 ? NKV - NQ : 0;
        q_row0 = int64_t(first) * p.H_Q + hq;
        q_stride = p.H_Q * D;
    }
    // causal workgroups cost what their position is: the late (long) ones are handed out first, so that the short
    // ones fill the end of the launch
    const int pos_block = p.causal ? int(gridDim.x) - 1 - int(blockIdx.x) : int(blockIdx.x);
    const int pos_first = (two_heads ? 64 : 128) * pos_block;            // of the workgroup
    if (pos_first >= NQ) return;                      // uniform: the grid is sized for the longest sequence
    const int pos_wg = two_heads ? pos_first : pos_first + 64 * wg;       // of this group (may lie beyond the sequence:
                                                                          // its rows are then computed and not stored)
    const int pos0 = pos_wg + 16 * wl;                // first row of this wavefront

    {   // threads 0..255 fill the key table, 256..511 the value table: entry tid % 256, all its copies
        const int e = tid & 255;
        const float* cen = tid < 256 ? p.centroids_k : p.centroids_v;
        const half2v c2 = {_Float16(cen[e >> 4]), _Float16(cen[e & 15])};
        const uint32_t bits = __builtin_bit_cast(uint32_t, c2);
        uint32_t* row = (tid < 256 ? pair_k : pair_v) + e * C::COPIES;
#pragma unroll
        for (int k = 0; k < C::COPIES; k += 4) *reinterpret_cast<uint4v*>(row + k) = uint4v{bits, bits, bits, bits};
    }

    // ---- rotate the 16 query rows of this wavefront, round to the query dtype, stage as fp16 ------
    float up = 1.0f;
    {
        int pos = pos0 + n16;
        pos = pos < NQ ? pos : NQ - 1;
        const uint16_t* src = p.q + (q_row0 * D) + int64_t(pos) * q_stride;
        // The 16-bit rows are exact in fp16 after one power of two for the block, the matrix block goes in as two
        // fp16 terms: exact products on the fp16 MFMA, at 8 times the rate of the float32 one (at head_dim 256 the
        // two rotations of a workgroup on the float32 MFMA took as long as 100 tiles of the loop).
        uint4v raw[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) raw[j] = *reinterpret_cast<const uint4v*>(src + 32 * j + 8 * g4);
        half8 ah[NJ];
        float up_rows;
        rows_as_f16<D, DT>(raw, ah, up_rows);
        float qr[NCB][4];
        float mx = 0.0f;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            float rb[NJ][8];
            load_rotation_any<D>(p.rotation, p.rot_col_major != 0, true, 16 * cb, n16, g4, rb);
            half8 rhi[NJ], rlo[NJ];
            split_rotation_block<D>(rb, rhi, rlo);
            const float4v acc = rotate_block_f16<D>(ah, rhi, rlo) * up_rows;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                qr[cb][i] = load_elem<DT>(store_elem<DT>(acc[i]));
                mx = __builtin_fmaxf(mx, __builtin_fabsf(qr[cb][i]));
            }
        }
        // one power of two for the wavefront's 16 rows, so that the rounded values are exact in fp16
        mx = wave_max(mx);
        int ex = int((float_to_bits(mx) >> 23) & 0xffu) - 127;
        if (ex < -100 || ex > 100) ex = 0;
        const float down = bits_to_float(uint32_t(127 - ex) << 23);
        up = bits_to_float(uint32_t(127 + ex) << 23);
        _Float16* mine = qs + w * 16 * C::KSTRIDE;
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
            for (int i = 0; i < 4; ++i) mine[(4 * g4 + i) * C::KSTRIDE + 16 * cb + n16] = _Float16(qr[cb][i] * down);
    }
    __syncthreads();
    half8 qa[NJ];
#pragma unroll
    for (int j = 0; j < NJ; ++j)
        qa[j] = *reinterpret_cast<const half8*>(qs + (w * 16 + n16) * C::KSTRIDE + 32 * j + 8 * g4);
    const float qscale = p.scale_log2e * up;
    __syncthreads();                                   // the query rows lie where the tiles go

    // ---- tiles --------------------------------------------------------------------------------------
    const int all_tiles = (NKV + 31) >> 5;
    int ntiles = all_tiles;
    if (p.causal) {
        const int span = two_heads ? 63 : 127;         // uniform over the workgroup: every wavefront meets every barrier
        int last_pos = pos_first + span < NQ - 1 ? pos_first + span : NQ - 1;
        const int t = ((qoff + last_pos) >> 5) + 1;
        ntiles = t < all_tiles ? t : all_tiles;
    }
    float4v O[NCB];
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) O[cb] = float4v{0.f, 0.f, 0.f, 0.f};
    float m_run[4], l_run[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) { m_run[i] = -__builtin_inff(); l_run[i] = 0.0f; }

    // dequantisation: token pair of the tile, 1 / 32 of its coordinates.  A wavefront takes 4 token pairs x 16 parts,
    // so that its transposed V stores (below) reach all banks
    const int tp = (lane >> 4) + 4 * (w >> 1), part = (lane & 15) + 16 * (w & 1);
    const int64_t k_row0 = PAGED ? 0 : (int64_t(b) * p.H_KV + hkv) * p.k_cap;
    const int64_t v_row0 = PAGED ? 0 : (int64_t(b) * p.H_KV + hkv) * p.v_cap;
    _Float16* pw = ps + w * 16 * C::VSTRIDE;

    // The packed bytes and norms of a tile are asked for one tile ahead (into registers), so that the
    // memory latency runs under the products of the tile before.
    uint32_t kw[2][1] = {{0u}, {0u}}, vw[2][1] = {{0u}, {0u}};
    float nk[2] = {0.0f, 0.0f}, nv[2] = {0.0f, 0.0f};
    auto load_tile = [&](int tile) {
        const int t0 = tile * 32;
        const uint8_t *kp[2], *vp[2];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            int tok = t0 + 2 * tp + u;
            const bool live = tok < NKV;
            tok = live ? tok : (NKV > 0 ? NKV - 1 : 0);
            if (PAGED) {
                const int H = p.H_KV;
                int pg = p.block_table[int64_t(b) * p.max_blocks + (tok >> p.bs_log2)];
                pg = pg < 0 ? 0 : (pg >= p.num_blocks ? p.num_blocks - 1 : pg);
                const uint8_t* row = p.cache + ((int64_t(pg) << p.bs_log2) + (tok & ((1 << p.bs_log2) - 1))) * (int64_t(H) * (D + 8));
                kp[u] = row + hkv * (D / 2);
                nk[u] = *reinterpret_cast<const float*>(row + H * (D / 2) + 4 * hkv);
                vp[u] = row + H * (D / 2 + 4) + hkv * (D / 2);
                nv[u] = *reinterpret_cast<const float*>(row + H * (D + 4) + 4 * hkv);
            } else {
                kp[u] = p.k_packed + (k_row0 + tok) * (D / 2);
                vp[u] = p.v_packed + (v_row0 + tok) * (D / 2);
                nk[u] = p.k_norms[k_row0 + tok];
                nv[u] = p.v_norms[v_row0 + tok];
            }
            if (!live) { nk[u] = 0.0f; nv[u] = 0.0f; }
            // packed bytes part * BPT .. of the token (BPT = 1, 2 or 4)
            if (BPT == 1) {
                kw[u][0] = kp[u][part];
                vw[u][0] = vp[u][part];
            } else if (BPT == 2) {
                kw[u][0] = *reinterpret_cast<const uint16_t*>(kp[u] + 2 * part);
                vw[u][0] = *reinterpret_cast<const uint16_t*>(vp[u] + 2 * part);
            } else {
                kw[u][0] = *reinterpret_cast<const uint32_t*>(kp[u] + 4 * part);
                vw[u][0] = *reinterpret_cast<const uint32_t*>(vp[u] + 4 * part);
            }
        }
    };
    if (ntiles > 0) load_tile(0);

    for (int tile = 0; tile < ntiles; ++tile) {
        const int t0 = tile * 32;
        // ---- dequantise: thread = (two consecutive tokens, D/16 coordinates of each) ---------------------
        {
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const int ek = norm_excess(nk[u]), ev = norm_excess(nv[u]);
                nk[u] = __builtin_ldexpf(nk[u], -ek);
                nv[u] = __builtin_ldexpf(nv[u], -ev);
                if (part == 0) { k_exc[2 * tp + u] = ek; v_exc[2 * tp + u] = ev; }
            }
            // K, row-major: byte j of the thread's run -> coordinates 2 (part BPT + j), + 1 of its token:
            // fp16(centroid) * norm, rounded to fp16 (the same values as the tuned kernel's tiles)
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                const _Float16 hn = _Float16(nk[u]);
                const half2v n2 = {hn, hn};
                uint32_t* dst = reinterpret_cast<uint32_t*>(ks + (2 * tp + u) * C::KSTRIDE + 2 * BPT * part);
                uint32_t wd[BPT];
#pragma unroll
                for (int j = 0; j < BPT; ++j) {
                    const uint32_t byte = (kw[u][j >> 2] >> (8 * (j & 3))) & 0xffu;
                    const half2v c2 = __builtin_bit_cast(half2v, pair_k[byte * C::COPIES + copy]) * n2;
                    wd[j] = __builtin_bit_cast(uint32_t, c2);
                }
                // the thread's run of the row in 8- or 16-byte stores (single dwords from 64 lanes that lie 16
                // to 32 bytes apart fall into a few banks)
                if constexpr (BPT == 1) {
                    *dst = wd[0];
                } else if constexpr (BPT == 2) {
                    *reinterpret_cast<uint2v*>(dst) = uint2v{wd[0], wd[1]};
                } else {
                    *reinterpret_cast<uint4v*>(dst) = uint4v{wd[0], wd[1 % BPT], wd[2 % BPT], wd[3 % BPT]};
                }
            }
            // V, transposed: a 2 x 2 nibble transpose makes a byte hold one coordinate of the two tokens,
            // so one lookup yields the dword (token 2 tp, token 2 tp + 1) of a coordinate row
            {
                const half2v n2 = {_Float16(nv[0]), _Float16(nv[1])};
                // The rows of the threads of a token pair lie 2 BPT rows apart, a multiple of 32 banks at 256
                // coordinates: with the pair's own column every one of their stores would hit the same bank.
                // The groups of four columns (8 tokens, what an operand read takes) are rotated by the thread's
                // part, and the parts walk through their coordinates in rotated order (a row further is 8 banks
                // further): the 64 lanes of a store (4 token pairs x 16 parts) fall two to a bank, the minimum.
                const int vcol = (tp + 4 * part) & 15;
                constexpr int JN = BPT < 4 ? BPT : 4;
#pragma unroll
                for (int c = 0; c < (BPT + 3) / 4; ++c) {
                    const uint32_t X = (vw[0][c] & 0xF0F0F0F0u) | ((vw[1][c] >> 4) & 0x0F0F0F0Fu);   // even coordinates
                    const uint32_t Y = ((vw[0][c] << 4) & 0xF0F0F0F0u) | (vw[1][c] & 0x0F0F0F0Fu);   // odd coordinates
#pragma unroll
                    for (int j0 = 0; j0 < JN; ++j0) {
                        const int j = (j0 + (part >> 2)) & (JN - 1);
                        const int d = 2 * (BPT * part + 4 * c + j);
                        const half2v xe = __builtin_bit_cast(half2v, pair_v[((X >> (8 * j)) & 0xffu) * C::COPIES + copy]) * n2;
                        const half2v yo = __builtin_bit_cast(half2v, pair_v[((Y >> (8 * j)) & 0xffu) * C::COPIES + copy]) * n2;
                        *reinterpret_cast<uint32_t*>(vt + d * C::VSTRIDE + 2 * vcol) = __builtin_bit_cast(uint32_t, xe);
                        *reinterpret_cast<uint32_t*>(vt + (d + 1) * C::VSTRIDE + 2 * vcol) = __builtin_bit_cast(uint32_t, yo);
                    }
                }
            }
        }
        __syncthreads();
        if (tile + 1 < ntiles) load_tile(tile + 1);

        // ---- scores: two blocks of 16 tokens ----------------------------------------------------------
        float4v s[2];
#pragma unroll
        for (int tb = 0; tb < 2; ++tb) {
            s[tb] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < NJ; ++j) {
                const half8 kb = *reinterpret_cast<const half8*>(ks + (16 * tb + n16) * C::KSTRIDE + 32 * j + 8 * g4);
                s[tb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(qa[j], kb, s[tb], 0, 0, 0);
            }
        }
        // lane (n16, g4): rows 4 g4 + i, tokens t0 + n16 and t0 + 16 + n16
        float pv[2][4];
        float alphas[4];
        bool moved = false;
        const int kx[2] = {k_exc[n16], k_exc[16 + n16]}, vx[2] = {v_exc[n16], v_exc[16 + n16]};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int qpos = qoff + pos0 + 4 * g4 + i;
            float sc[2];
            float mx = -__builtin_inff();
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) {
                const int tok = t0 + 16 * tb + n16;
                const bool ok = tok < NKV && (!p.causal || tok <= qpos);
                sc[tb] = ok ? __builtin_ldexpf(s[tb][i] * qscale, kx[tb]) : -__builtin_inff();
                // the reference is taken over score + value excess: weight * 2^excess then stays <= 1
                mx = __builtin_fmaxf(mx, sc[tb] + float(vx[tb]));
            }
            mx = row16_max(mx);
            const float m_new = __builtin_fmaxf(m_run[i], mx);
            const float m_use = m_new == -__builtin_inff() ? 0.0f : m_new;
            const float alpha = __builtin_amdgcn_exp2f(m_run[i] - m_use);
            m_run[i] = m_new;
            float rs = 0.0f;
#pragma unroll
            for (int tb = 0; tb < 2; ++tb) {
                pv[tb][i] = __builtin_amdgcn_exp2f(sc[tb] - m_use);
                rs += pv[tb][i];
            }
            l_run[i] = __builtin_fmaf(l_run[i], alpha, rs);     // per-lane partial; summed over the row at the end
            alphas[i] = alpha;
            moved = moved || alpha != 1.0f;
        }
        // the accumulators are rescaled only when some row's maximum moved (after the first tiles it rarely does)
        if (__any(moved)) {
#pragma unroll
            for (int cb = 0; cb < NCB; ++cb)
#pragma unroll
                for (int i = 0; i < 4; ++i) O[cb][i] *= alphas[i];
        }
        // P (C layout) -> LDS patch -> A layout
#pragma unroll
        for (int tb = 0; tb < 2; ++tb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                pw[(4 * g4 + i) * C::VSTRIDE + 16 * tb + n16] = _Float16(__builtin_ldexpf(pv[tb][i], vx[tb]));
        const half8 pa = *reinterpret_cast<const half8*>(pw + n16 * C::VSTRIDE + 8 * g4);
#pragma unroll
        for (int cb = 0; cb < NCB; ++cb) {
            // (the column groups of a row are rotated by the index of the thread that wrote it: row / (2 BPT))
            const int vrow = 16 * cb + n16;
            const half8 vb = *reinterpret_cast<const half8*>(vt + vrow * C::VSTRIDE + 8 * ((g4 + vrow / (2 * BPT)) & 3));
            O[cb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, vb, O[cb], 0, 0, 0);
        }
        __syncthreads();                               // the tiles are free again
    }

    // ---- normalise, rotate back, store ------------------------------------------------------------------
    // The staging rows overlay the tiles, a patch per wavefront that only its own lanes write and read; the two
    // groups of four wavefronts take the patches one after the other.
    float* os = reinterpret_cast<float*>(smem) + wl * 16 * (D + 4);
    float a[NJ][8];
#pragma unroll
    for (int round = 0; round < 2; ++round) {
        __syncthreads();                               // the tiles (round 0), the other group's patches (round 1) are free
        if (wg == round) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float l = row16_sum(l_run[i]);
                const float inv = l > 0.0f ? 1.0f / l : 0.0f;
#pragma unroll
                for (int cb = 0; cb < NCB; ++cb) {
                    float v = O[cb][i] * inv;
                    if (PAGED) v = load_elem<DT>(store_elem<DT>(v));
                    os[(4 * g4 + i) * (D + 4) + 16 * cb + n16] = v;
                }
            }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int j = 0; j < NJ; ++j)
#pragma unroll
                for (int k = 0; k < 8; ++k) a[j][k] = os[n16 * (D + 4) + 32 * j + 8 * g4 + k];
        }
    }
    uint16_t* obase = p.out + q_row0 * D;
    // float32 rows as two fp16 terms (rows already rounded to the output type, the paged form: exact in one)
    half8 ohi[NJ], olo[NJ];
    float up_out;
    rows_split_f16<D>(a, ohi, olo, up_out);
#pragma unroll
    for (int cb = 0; cb < NCB; ++cb) {
        float rb[NJ][8];
        load_rotation_any<D>(p.rotation, p.rot_col_major != 0, false, 16 * cb, n16, g4, rb);
        half8 rhi[NJ], rlo[NJ];
        split_rotation_block<D>(rb, rhi, rlo);
        const float4v acc = (PAGED ? rotate_block_f16<D>(ohi, rhi, rlo) : rotate_block_f16x3<D>(ohi, olo, rhi, rlo)) * up_out;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int pos = pos0 + 4 * g4 + i;
            if (pos < NQ) obase[int64_t(pos) * q_stride + 16 * cb + n16] = store_elem<DT>(acc[i]);
        }
    }
}

template <int D, bool PAGED>
int launch_any_dim(const AnyDimParams& p, int max_q, int batch, int dtype, hipStream_t s) {
    const bool two_heads = (p.G & 1) == 0;            // as the kernel decides
    const dim3 grid(two_heads ? (max_q + 63) / 64 : (max_q + 127) / 128, two_heads ? p.H_Q / 2 : p.H_Q, batch), block(512);
    const size_t lds = AnyDimCfg<D>::LDS_BYTES;
    if (dtype == FQ_F16) {
        auto kern = tq_attention_any_dim_kernel<D, FQ_F16, PAGED>;
        if (lds > 32768 && !fq_host::lds_limit_raised(reinterpret_cast<const void*>(kern), lds)) return FQ_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, block, lds, s, p);
    } else {
        auto kern = tq_attention_any_dim_kernel<D, FQ_BF16, PAGED>;
        if (lds > 32768 && !fq_host::lds_limit_raised(reinterpret_cast<const void*>(kern), lds)) return FQ_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, block, lds, s, p);
    }
    return fq_host::check_launch();
}

// Entry for the two host functions of fq_fused_attention.hip: every argument already checked.
int launch_attention_any_dim(const AnyDimParams& p, int D, bool paged, int max_q, int batch, int dtype, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (p.H_Q > 65535 || batch > 65535) return FQ_ERR_BAD_SHAPE;
    switch (D) {
        case 64: return paged ? launch_any_dim<64, true>(p, max_q, batch, dtype, s) : launch_any_dim<64, false>(p, max_q, batch, dtype, s);
        case 128: return paged ? launch_any_dim<128, true>(p, max_q, batch, dtype, s) : launch_any_dim<128, false>(p, max_q, batch, dtype, s);
        case 256: return paged ? launch_any_dim<256, true>(p, max_q, batch, dtype, s) : launch_any_dim<256, false>(p, max_q, batch, dtype, s);
        default: return FQ_ERR_UNSUPPORTED_DIM;
    }
}

}  // namespace fq

namespace fq_host {
bool force_any_dim_attention() { return option(FQ_OPT_ATTENTION_ANY_DIM) != 0; }
}
