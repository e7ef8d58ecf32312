// Split-K paged decode from the packed TQ4 cache, gfx950.
//
// Operator: paged_decode_reference (src/flashquant/kernels/cpu_reference.py:230-368)
// wrapped by the query pre-rotation and output post-rotation of
// src/flashquant/kernels/paged_decode.py:112-128.  Token row of the cache:
// [K idx H*D/2 | K norm H*4 | V idx H*D/2 | V norm H*4] (src/flashquant/vllm/impl.py:132-138).
//
// Launches on the caller's stream:
//   rotate_q_kernel              q_rot = (q @ R^T) rounded to the query dtype; only for
//                                shapes whose decode kernel does not rotate the query itself
//   paged_decode_staged_kernel   8 KV heads of 128 coordinates: one workgroup per (split,
//                                sequence); 4 wavefronts copy whole token rows to LDS and
//                                wavefront h of 8 more works on KV head h; rotates the query
//                                in its prologue; also serves TurboQuantProd pages
//   paged_decode_kernel          every other shape: one wavefront per (split, sequence, KV
//                                head), operands read straight from global memory
//   reduce_rotate_kernel         log-sum-exp combine of the split partials (m, l, acc[D]),
//                                rounded to the query dtype, then (out_rot @ R) rounded again
//
// The decode kernels are bound by HBM traffic (136 bytes per token per KV head) only
// if the per-byte work is small: with 4 query heads per KV head, float32 FMAs alone
// would cost more than the memory time, so both products run on the 16x16x32 fp16
// MFMA and the dequantisation is one LDS lookup per packed byte: a 256-entry table maps
// a byte to the fp16 pair (centroid[hi nibble], centroid[lo nibble]), replicated so
// that the lanes of a half-wave always read different banks whatever the data.
//
// Per 16-token block:
//   scores   S^T_blk = K_blk (16 tokens x D) . Q^T (D x 16 columns).  Column n
//            carries query head n % GP (GP = group size padded to 4, 8 or 16), so
//            every block's result holds each head 16/GP times; lane (n, g) keeps
//            the copy of block class n / GP.  After that selection a lane owns
//            consecutive tokens of one head per kept block, all lanes busy.
//            A lane's K operand is the 16 bytes it loaded (token n, quarter g of
//            the row): the contraction index is permuted (k-step ks, group g,
//            element e) <-> d = g*D/4 + 8*ks + e, and Q is loaded the same way.
//   softmax  base 2, float32; the weight handed to the second product is w * |v| in
//            fp16 (the V norm rides on the weight), the denominator accumulates w.  The
//            running reference moves only when a score leads it by more than 2^16 or a
//            product w * |v| would pass 60000; it then becomes the maximum over the tile
//            of score + (binary orders of |v| above 2^10), so the product stays below
//            2^11 whatever the norms are and accumulator rescales are rare.
//   output   O (16 rows x D) += P (16 x tokens) . V (tokens x D), where row n of P
//            holds the weights of head n % GP for the tokens of block class n / GP
//            only (zero elsewhere), so the lane that computed a weight is the lane
//            that feeds it to the MFMA: no cross-lane movement.  The classes are
//            summed once per split.  V's contraction index is the token, so a lane
//            loads the bytes of D/16 consecutive coordinates (lane n <-> d = n*D/16
//            ...) of its tokens, and a 2x2 nibble transpose of token pairs makes
//            each byte hold the same coordinate of two consecutive tokens: again
//            one lookup per byte.

#include <cstdlib>
#include <map>
#include <mutex>
#include <utility>

#include "fq_common.hpp"
#include "fq_device.hpp"
#include "fq_paged_decode.hpp"

namespace fq_host {
int device_cu_count();
}

namespace fq {




// head_dim 256 keeps 64 accumulator registers per lane and runs with at most four wavefronts per workgroup,
// so that a wavefront may use up to 512 registers (with eight it spilled 150-220 of them).
template <int D, int BSL, int GP, int DT, int PVR>
__global__ __launch_bounds__(D == 256 ? 256 : 512) void paged_decode_kernel(const DecodeParams p) {
    constexpr int BS = 1 << BSL;
    constexpr int KS = D / 32;            // k-steps of the score product
    constexpr int KW = D / 32;            // K dwords per lane per block
    constexpr int DPL = D / 16;           // V coordinates per lane
    constexpr int VW = DPL > 8 ? 2 : 1;   // V dwords per lane per token
    constexpr int NB = 16 / GP;           // block classes
    constexpr int NC = 4 / NB;            // kept blocks per lane per tile
    constexpr int ROW_HALF = D / 2;

    __shared__ __attribute__((aligned(256))) uint32_t lut[kLutWords];   // K table (static: constant LDS address)
    extern __shared__ uint32_t lut2[];                                  // V table when it differs

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int waves = blockDim.x >> 6;
    const int n = lane & 15;
    const int g = lane >> 4;
    const int hd = n % GP;                // query head inside the group
    const int bc_lane = n / GP;           // block class kept by this lane
    // Fewer KV heads than wavefronts: the workgroup serves all heads of waves / heads_per_wg consecutive
    // splits (a workgroup of one or two wavefronts would leave the CU, which holds two such workgroups
    // beside their 64 KB tables, almost empty).
    const int split = int(blockIdx.x) * (waves / p.heads_per_wg) + wave / p.heads_per_wg;
    const int seq = blockIdx.y;
    const int h = blockIdx.z * p.heads_per_wg + wave % p.heads_per_wg;

    // ---- byte -> (fp16, fp16) tables, one copy per LDS bank ----------------------
    build_byte_table(lut, p.centroids_k, wave, waves, lane);
    if (p.two_tables) build_byte_table(lut2, p.centroids_v, wave, waves, lane);
    __syncthreads();
    if (h >= p.H_KV || split >= p.num_splits) return;
    const uint8_t* lut_k = reinterpret_cast<const uint8_t*>(lut);
    const uint8_t* lut_v = p.two_tables ? reinterpret_cast<const uint8_t*>(lut2) : lut_k;
    const uint32_t lane_off = 4u * lane;

    int L = p.seq_lens[seq];
    L = L < 0 ? 0 : L;
    L = L > p.max_blocks * BS ? p.max_blocks * BS : L;
    const int NS = p.num_splits;
    // every sequence is cut into the same token chunks (those of the longest possible context):
    // the work of a workgroup does not depend on its sequence's length, short sequences just
    // leave their last splits empty
    const int chunk = (((p.max_blocks * BS + NS - 1) / NS) + 63) & ~63;
    const int begin = split * chunk;
    const int end = L < begin + chunk ? L : begin + chunk;

    const int hq_lane = h * p.G + n;      // for lanes n < G: the query head whose m, l they publish
    if (begin >= end) {
        if (g == 0 && n < p.G) {
            const int64_t o = (int64_t(seq) * p.H_Q + hq_lane) * NS + split;
            p.part_m[o] = -__builtin_inff();
            p.part_l[o] = 0.0f;
        }
        return;
    }

    const int row_bytes = p.H_KV * (D + 8);
    const int k_norm_off = p.H_KV * ROW_HALF + 4 * h;
    const int v_idx_off = p.H_KV * (ROW_HALF + 4) + h * ROW_HALF;
    const int v_norm_off = p.H_KV * (D + 4) + 4 * h;
    const int32_t* bt = p.block_table + int64_t(seq) * p.max_blocks;
    const int last_page_idx = (L - 1) >> BSL;

    // ---- the query of this lane's head, as the B operand of the score product ----
    half8 qh[KS];
    float qscale;
    {
        float qf[KS][8];
        float mx = 0.0f;
        const bool live = hd < p.G;
        const uint16_t* qsrc = reinterpret_cast<const uint16_t*>(p.q_rot) +
                               (int64_t(seq) * p.H_Q + h * p.G + (live ? hd : 0)) * D + g * (D / 4);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            const uint4v raw = *reinterpret_cast<const uint4v*>(qsrc + 8 * ks);
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                qf[ks][2 * i] = live ? load_elem<DT>(uint16_t(w[i] & 0xffffu)) : 0.0f;
                qf[ks][2 * i + 1] = live ? load_elem<DT>(uint16_t(w[i] >> 16)) : 0.0f;
                mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(qf[ks][2 * i]), __builtin_fabsf(qf[ks][2 * i + 1])));
            }
        }
        mx = max_xor32(max_xor16(mx));
        int ex = int((float_to_bits(mx) >> 23) & 0xffu) - 127;
        if (ex < -100 || ex > 100) ex = 0;
        const float down = bits_to_float(uint32_t(127 - ex) << 23);
        qscale = p.scale_log2e * bits_to_float(uint32_t(127 + ex) << 23);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) qh[ks][e] = _Float16(qf[ks][e] * down);
    }

    // ---- per-tile register image ----------------------------------------------
    struct Tile {
        uint32_t k[4][KW];
        uint32_t v[2][8][VW];
        float kn[NC][4];
        float vn[NC][4];
    };

    const uint8_t* cache = p.cache;
    const int max_page = p.num_blocks - 1;
    const int64_t page_bytes = int64_t(BS) * row_bytes;

    // Lane-constant byte offsets from the base of a block's page: the K operand
    // reads row n (quarter g of the head's index bytes), the V operand and the
    // norms read rows 4g + 0..3.  With 8-token pages a 16-token block spans two
    // pages and rows 8..15 live in the second one (k_hi / r_hi).
    constexpr bool SMALL_PAGES = BSL == 3;
    const bool k_hi = SMALL_PAGES && (n & 8);
    const bool r_hi = SMALL_PAGES && (g & 2);
    const uint32_t k_off = uint32_t((SMALL_PAGES ? (n & 7) : n) * row_bytes + h * ROW_HALF + g * (D / 8));
    uint32_t v_off[4], n_off[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int r = SMALL_PAGES ? ((4 * g + i) & 7) : 4 * g + i;
        v_off[i] = uint32_t(r * row_bytes + v_idx_off + n * (DPL / 2));
        n_off[i] = uint32_t(r * row_bytes + k_norm_off);
    }
    const uint32_t vn_delta = uint32_t(v_norm_off - k_norm_off);

    // Page ids of this split, fetched once: lane i of register r holds the page of
    // split-local page index 64 r + i (clamped to the sequence's last page and to the
    // cache size, so every address formed from them stays inside the cache).  A tile
    // then gets its pages with v_readlane, with no memory access on its critical path.
    int pv[PVR];
    const int split_p0 = begin >> BSL;
#pragma unroll
    for (int r = 0; r < PVR; ++r) {
        int idx = split_p0 + 64 * r + lane;
        idx = idx > last_page_idx ? last_page_idx : idx;
        int pg = bt[idx];
        pv[r] = pg < 0 ? 0 : (pg > max_page ? max_page : pg);
    }
    auto page_id = [&](int rel) -> int {   // rel: split-local page index, wave-uniform
        int v = __builtin_amdgcn_readlane(pv[0], rel & 63);
#pragma unroll
        for (int r = 1; r < PVR; ++r) {
            const int vr = __builtin_amdgcn_readlane(pv[r], rel & 63);
            v = (rel >> 6) == r ? vr : v;
        }
        return v;
    };

    // Loads one tile.  Tokens at or past `end` are not clamped: their values are
    // masked later.
    auto load_tile = [&](int t0, Tile& t) {
        const uint8_t* lo[4];
        const uint8_t* hi[4];
        const int p0 = (t0 >> BSL) - split_p0;
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            const int rel = BSL == 4 ? blk : (BSL == 5 ? (blk >> 1) : 2 * blk);
            lo[blk] = cache + int64_t(page_id(p0 + rel)) * page_bytes + ((BSL == 5 && (blk & 1)) ? 16 * row_bytes : 0);
            hi[blk] = SMALL_PAGES ? cache + int64_t(page_id(p0 + rel + 1)) * page_bytes : lo[blk];
        }
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            const uint8_t* src = (k_hi ? hi[blk] : lo[blk]) + k_off;
            if constexpr (KW == 4) {
                const uint4v w = *reinterpret_cast<const uint4v*>(src);
                t.k[blk][0] = w.x; t.k[blk][1] = w.y; t.k[blk][2] = w.z; t.k[blk][3] = w.w;
            } else if constexpr (KW == 2) {
                const uint2v w = *reinterpret_cast<const uint2v*>(src);
                t.k[blk][0] = w.x; t.k[blk][1] = w.y;
            } else {
#pragma unroll
                for (int q4 = 0; q4 < KW / 4; ++q4) {
                    const uint4v w = *reinterpret_cast<const uint4v*>(src + 16 * q4);
                    t.k[blk][4 * q4] = w.x; t.k[blk][4 * q4 + 1] = w.y;
                    t.k[blk][4 * q4 + 2] = w.z; t.k[blk][4 * q4 + 3] = w.w;
                }
            }
        }
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int blk = 2 * ks + j / 4;
                const uint8_t* src = (r_hi ? hi[blk] : lo[blk]) + v_off[j % 4];
                if (DPL == 4) {
                    t.v[ks][j][0] = *reinterpret_cast<const uint16_t*>(src);
                } else if (DPL == 8) {
                    t.v[ks][j][0] = *reinterpret_cast<const uint32_t*>(src);
                } else {
                    const uint2v w = *reinterpret_cast<const uint2v*>(src);
                    t.v[ks][j][0] = w.x;
                    t.v[ks][j][VW - 1] = w.y;
                }
            }
        }
#pragma unroll
        for (int c = 0; c < NC; ++c) {
            const uint8_t* base = r_hi ? hi[c * NB] : lo[c * NB];
#pragma unroll
            for (int bc = 1; bc < NB; ++bc) base = bc_lane == bc ? (r_hi ? hi[c * NB + bc] : lo[c * NB + bc]) : base;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                t.kn[c][i] = *reinterpret_cast<const float*>(base + n_off[i]);
                t.vn[c][i] = *reinterpret_cast<const float*>(base + n_off[i] + vn_delta);
            }
        }
    };

    // ---- running state ----------------------------------------------------------
    float4v O[DPL];
#pragma unroll
    for (int db = 0; db < DPL; ++db) O[db] = float4v{0.f, 0.f, 0.f, 0.f};
    float M = -__builtin_inff();
    float lsum = 0.0f;

    constexpr int VG = DPL / 4;      // groups of four coordinate blocks per k-step of P.V

    auto compute_tile = [&](int t0, const Tile& cur) {
        // The LDS lookups of one group of operands are issued before the MFMAs of the
        // previous group, so that the LDS latency overlaps matrix work; the scheduling
        // fences keep the compiler from serialising lookup -> wait -> MFMA again.
        uint4v ka[2][KS];
        auto k_group = [&](int blk, uint4v (&dst)[KS]) {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint32_t w = cur.k[blk][ks];
                dst[ks] = lookup_word(lut_k, w, lane_off);
            }
        };
        // nibble transposes of the V token pairs (all of them: 2 k-steps x 4 pairs)
        uint32_t X[2][4][VW], Y[2][4][VW];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int jp = 0; jp < 4; ++jp)
#pragma unroll
                for (int wv = 0; wv < VW; ++wv) {
                    const uint32_t A = cur.v[ks][2 * jp][wv], B = cur.v[ks][2 * jp + 1][wv];
                    X[ks][jp][wv] = (A & 0xF0F0F0F0u) | ((B >> 4) & 0x0F0F0F0Fu);
                    Y[ks][jp][wv] = ((A << 4) & 0xF0F0F0F0u) | (B & 0x0F0F0F0Fu);
                }
        uint4v vb[2][4];
        auto v_group = [&](int grp, uint4v (&dst)[4]) {   // grp = ks * VG + quarter
            const int ks = grp / VG, q4 = grp % VG;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int db = 4 * q4 + e, bi = db / 2;
                const uint32_t (&src)[4][VW] = (db & 1) ? Y[ks] : X[ks];
                const uint32_t col[4] = {src[0][bi / 4], src[1][bi / 4], src[2][bi / 4], src[3][bi / 4]};
                dst[e] = (bi % 4 == 0) ? lookup_column<0>(lut_v, col, lane_off)
                       : (bi % 4 == 1) ? lookup_column<1>(lut_v, col, lane_off)
                       : (bi % 4 == 2) ? lookup_column<2>(lut_v, col, lane_off)
                                       : lookup_column<3>(lut_v, col, lane_off);
            }
        };

        // ---- scores --------------------------------------------------------------
        float s_[NC][4];
        k_group(0, ka[0]);
#pragma unroll
        for (int blk = 0; blk < 4; ++blk) {
            if (blk < 3) k_group(blk + 1, ka[(blk + 1) & 1]);
            else v_group(0, vb[0]);
            __builtin_amdgcn_sched_barrier(0);
            float4v acc = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ka[blk & 1][ks]), qh[ks], acc, 0, 0, 0);
            const int c = blk / NB, bc = blk % NB;
#pragma unroll
            for (int i = 0; i < 4; ++i) s_[c][i] = (bc == 0 || bc_lane == bc) ? acc[i] : s_[c][i];
            __builtin_amdgcn_sched_barrier(0);
        }

        float a_[NC][4], rv[NC][4];   // rv: value norm of a live token, 0 for a masked one
        float tmax = -__builtin_inff();
#pragma unroll
        for (int c = 0; c < NC; ++c) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int tok = t0 + 16 * (c * NB + bc_lane) + 4 * g + i;
                const bool live = tok < end;
                rv[c][i] = live ? cur.vn[c][i] : 0.0f;
                a_[c][i] = live ? s_[c][i] * cur.kn[c][i] * qscale : -__builtin_inff();
                // the bias (0 for ordinary value norms) keeps weight * norm inside fp16
                tmax = __builtin_fmaxf(tmax, a_[c][i] + norm_bias(rv[c][i]));
            }
        }
        tmax = max_same_head<GP>(tmax);
        const float Mnew = __builtin_fmaxf(M, tmax);
        const float Ms = Mnew == -__builtin_inff() ? 0.0f : Mnew;
        const float alpha = __builtin_amdgcn_exp2f(M - Ms);
        M = Mnew;

        _Float16 wh[NC][4];
        float psum = 0.0f;
#pragma unroll
        for (int c = 0; c < NC; ++c) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float w = __builtin_amdgcn_exp2f(a_[c][i] - Ms);
                psum += w;
                wh[c][i] = _Float16(__builtin_fminf(w * rv[c][i], kHalfMax));
            }
        }
        lsum = __builtin_fmaf(lsum, alpha, psum);

        // ---- rescale the accumulators when a maximum moved --------------------------
        if (__any(alpha != 1.0f)) {
            float ar[4];
            if (GP == 4) {
                // row 4g + i belongs to head i, held by the lane at position i of this lane's quad
                ar[0] = dpp_mov<0x00>(alpha);
                ar[1] = dpp_mov<0x55>(alpha);
                ar[2] = dpp_mov<0xAA>(alpha);
                ar[3] = dpp_mov<0xFF>(alpha);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) ar[i] = __shfl(alpha, 4 * g + i, kWave);
            }
#pragma unroll
            for (int db = 0; db < DPL; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) O[db][i] *= ar[i];
        }

        // ---- weights as the A operand: row n feeds only its own block class -------------
        half8 pa[2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int hf = 0; hf < 2; ++hf) {
                constexpr _Float16 zero = _Float16(0.0f);
                const int blk = 2 * ks + hf;
                const int c = blk / NB, bc = blk % NB;
                const bool mine = bc_lane == bc;
#pragma unroll
                for (int i = 0; i < 4; ++i) pa[ks][4 * hf + i] = mine ? wh[c][i] : zero;
            }
        }

        // ---- O += P . V, lookups of the next group in flight during the MFMAs ------------
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int grp = 0; grp < 2 * VG; ++grp) {
            if (grp + 1 < 2 * VG) v_group(grp + 1, vb[(grp + 1) & 1]);
            __builtin_amdgcn_sched_barrier(0);
            const int ks = grp / VG, q4 = grp % VG;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                O[4 * q4 + e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa[ks], __builtin_bit_cast(half8, vb[grp & 1][e]),
                                                                      O[4 * q4 + e], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- tiles of the split, two register images in ping-pong ------------------------
    // The prefetch of the next tile is unconditional (past the last tile it reloads
    // the last one): a branch around it would make the compiler wait for every
    // outstanding load where the paths merge, which serialises load and compute.
    // The workgroup barrier keeps the wavefronts (one per KV head) on the same tile,
    // so that the halves of a cache line that two heads share are asked for together.
    {
        Tile ta, tb;
        int t0 = begin;
        const int last_t0 = begin + ((end - begin - 1) & ~63);
        load_tile(t0, ta);
        while (true) {
            __builtin_amdgcn_s_barrier();
            load_tile(t0 + 64 < last_t0 ? t0 + 64 : last_t0, tb);
            compute_tile(t0, ta);
            t0 += 64;
            if (t0 >= end) break;
            __builtin_amdgcn_s_barrier();
            load_tile(t0 + 64 < last_t0 ? t0 + 64 : last_t0, ta);
            compute_tile(t0, tb);
            t0 += 64;
            if (t0 >= end) break;
        }
    }

    // ---- publish the partial of this split --------------------------------------------
#pragma unroll
    for (int mask = GP; mask < 64; mask <<= 1) lsum += xor_shuffle(lsum, mask);
#pragma unroll
    for (int db = 0; db < DPL; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = O[db][i];
#pragma unroll
            for (int mask = 4 * GP; mask < 64; mask <<= 1) v += xor_shuffle(v, mask);
            O[db][i] = v;
        }
    if (g == 0 && n < p.G) {
        const int64_t o = (int64_t(seq) * p.H_Q + hq_lane) * NS + split;
        p.part_m[o] = M;
        p.part_l[o] = lsum;
    }
    if (g < GP / 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int head = 4 * g + i;
            if (head < p.G) {
                float* dst = p.part_acc + ((int64_t(seq) * p.H_Q + h * p.G + head) * NS + split) * D + n * DPL;
#pragma unroll
                for (int q4 = 0; q4 < DPL / 4; ++q4) {
                    const float4v v = {O[4 * q4][i], O[4 * q4 + 1][i], O[4 * q4 + 2][i], O[4 * q4 + 3][i]};
                    *reinterpret_cast<float4v*>(dst + 4 * q4) = v;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------------------
// Staged variant for 8 KV heads of dimension 128 (the common GQA layout).
//
// The direct kernel above lets every wavefront fetch its own head's bytes, which are
// 64-byte halves of cache lines it shares with the neighbouring head and 4-byte norms
// inside 32-byte strips shared by all heads: the vector L1 then spends its time on
// requests for lines that are already in flight.  Here the workgroup (8 computing
// wavefronts, one per KV head) copies whole token rows: a copying thread t of T moves the
// 16-byte chunks t, t + T, ... of a 32-token tile, so every wavefront request covers eight complete cache lines and
// each line is asked for exactly once.  The chunks land in LDS in a swizzled layout from
// which the wavefronts read their MFMA operands without bank conflicts:
//
//   stage (16 tokens) = [K idx 8 KB | V idx 8 KB | K norms 512 B | V norms 512 B]
//   16-byte slot of (head h, row r, quarter q) = 64 h + 4 p + (q ^ ((p >> 1) & 3)),
//   p = r ^ ((r >> 2) & 1) ^ (h & 1)
//
// (rows r and r + 4, read together by the P.V operand loads, fall in different halves of
// the banks; the eight rows read together by a K operand load fall in eight different
// 16-byte bank groups; the eight chunks a quarter-wave writes together do too).
//
// Pipeline.  With copy wavefronts (CW = 4, the default) four more wavefronts do nothing but
// move tiles: each keeps two tiles in flight in registers and writes a tile to an LDS slot as
// soon as the eight computing wavefronts have read the slot's previous tile into registers,
// which they do at the very start of a tile; the computing wavefronts never wait for global
// memory.  The two sides meet through counting flags in LDS (a bounded buffer of two slots), not
// through workgroup barriers, so no wavefront waits for one that it does not depend on.  Without
// copy wavefronts (CW = 0) the eight wavefronts do both, one workgroup barrier per tile: at
// iteration i the registers holding tile i + 1 (loaded during iteration i - 1) are written to the
// free slot, the loads of tile i + 2 are issued, and tile i is consumed from LDS.
// A tile is 32 tokens: two 16-token blocks; with 4 query heads per KV head the 16 MFMA
// columns carry (head, block, half of the block's rows), so that all lanes own distinct
// (head, token) scores.
// ---------------------------------------------------------------------------------------

// TurboQuantProd pages (PROD): the key nibble is (sign bit << 3 | 3-bit index) and a key
// carries a second float32, the residual norm, so a token row is
// [K nibbles H*64 | K norm H*4 | K residual norm H*4 | V idx H*64 | V norm H*4] = H*140 bytes
// and a stage grows by 512 bytes of residual norms.
// DIM = 64 (TQ4 pages): two neighbouring KV heads of 64 coordinates are served as one "head" of 128 (their index
// bytes are contiguous in the token row), with two norms each for K and V: a row of 8 such heads is 16 real
// heads, 72 chunks.  DIM = 256: a KV head of 256 coordinates is served as two "heads" of 128 (the halves of its
// index bytes) that share its norms: a row of 8 such heads is 4 real heads, 66 chunks.
template <bool PROD, int DIM = 128>
struct StagedCfg {
    static constexpr int CHUNKS_PER_ROW = PROD ? 70 : (DIM == 64 ? 72 : (DIM == 256 ? 66 : 68));   // 16-byte chunks of a row
    static constexpr int ROWB = 16 * CHUNKS_PER_ROW;               // 1088 / 1120 / 1152 / 1056
    static constexpr int STAGE_BYTES = 16 * ROWB;                  // 17408 / 17920 / 18432 / 16896
    static constexpr int TILE_BYTES = 2 * STAGE_BYTES;             // 32 tokens
    static constexpr int CHUNKS_PER_TILE = 32 * CHUNKS_PER_ROW;    // 2176 / 2240 / 2304 / 2112
    static constexpr int NORM_BYTES = DIM == 64 ? 64 : (DIM == 256 ? 16 : 32);   // K (or V) norms of a row
    static constexpr int KN_OFF = 16384;                           // K norms of the stage's 16 rows
    static constexpr int VN_OFF = KN_OFF + 16 * NORM_BYTES;        // V norms
};
constexpr int kStageKnOff = 16384;
constexpr int kStageVnOff = 16896;
constexpr int kStageKgOff = 17408;

__host__ __device__ constexpr int staged_slot(int h, int r, int q) {
    const int pp = (r ^ ((r >> 2) & 1) ^ (h & 1)) & 15;
    return 64 * h + 4 * pp + (q ^ ((pp >> 1) & 3));
}

// LDS byte offset (inside a tile slot) of the 16-byte chunk `ci` of tile row `row` (0..31).
template <bool PROD, int DIM = 128>
__host__ __device__ constexpr int staged_chunk_dst(int row, int ci) {
    const int stage = row >> 4, r = row & 15;
    int off = 0;
    if (DIM == 64) {
        using C = StagedCfg<false, 64>;
        if (ci < 32) off = 16 * staged_slot(ci >> 2, r, ci & 3);
        else if (ci < 36) off = C::KN_OFF + 64 * r + 16 * (ci - 32);
        else if (ci < 68) off = 8192 + 16 * staged_slot((ci - 36) >> 2, r, (ci - 36) & 3);
        else off = C::VN_OFF + 64 * r + 16 * (ci - 68);
        return stage * C::STAGE_BYTES + off;
    }
    if (DIM == 256) {
        using C = StagedCfg<false, 256>;
        if (ci < 32) off = 16 * staged_slot(ci >> 2, r, ci & 3);
        else if (ci == 32) off = C::KN_OFF + 16 * r;
        else if (ci < 65) off = 8192 + 16 * staged_slot((ci - 33) >> 2, r, (ci - 33) & 3);
        else off = C::VN_OFF + 16 * r;
        return stage * C::STAGE_BYTES + off;
    }
    if (ci < 32) {
        off = 16 * staged_slot(ci >> 2, r, ci & 3);
    } else if (ci < 34) {
        off = kStageKnOff + 32 * r + 16 * (ci - 32);
    } else if (PROD && ci < 36) {
        off = kStageKgOff + 32 * r + 16 * (ci - 34);
    } else {
        const int cv = ci - (PROD ? 36 : 34);
        if (cv < 32) off = 8192 + 16 * staged_slot(cv >> 2, r, cv & 3);
        else off = kStageVnOff + 32 * r + 16 * (cv - 32);
    }
    return stage * StagedCfg<PROD>::STAGE_BYTES + off;
}

// The same offsets for every chunk of a tile, worked out at compile time: a thread reads its
// five entries instead of dividing by the row length and walking the layout.
template <bool PROD, int DIM = 128>
struct ChunkDstTable {
    uint16_t off[StagedCfg<PROD, DIM>::CHUNKS_PER_TILE];
    constexpr ChunkDstTable() : off() {
        for (int c = 0; c < StagedCfg<PROD, DIM>::CHUNKS_PER_TILE; ++c)
            off[c] = uint16_t(staged_chunk_dst<PROD, DIM>(c / StagedCfg<PROD, DIM>::CHUNKS_PER_ROW,
                                                          c % StagedCfg<PROD, DIM>::CHUNKS_PER_ROW));
    }
};
template <bool PROD, int DIM = 128>
__device__ const ChunkDstTable<PROD, DIM> kChunkDst{};

// TurboQuantProd sign operand: the fp16 pairs (+-1, +-1) of the eight sign bits (bit 3 of
// every nibble) of one key dword.  Element e of the result belongs to the coordinate
// kSignOrder[e] of the dword's eight: the query-side operand is permuted to match.
__device__ __forceinline__ uint4v sign_operand(uint32_t w, uint32_t ones) {
    uint4v r;
    r.x = (w & 0x80008000u) | ones;
    r.y = ((w << 4) & 0x80008000u) | ones;
    r.z = ((w << 8) & 0x80008000u) | ones;
    r.w = ((w << 12) & 0x80008000u) | ones;
    return r;
}
__device__ __forceinline__ constexpr int sign_order(int e) {
    constexpr int order[8] = {2, 6, 3, 7, 0, 4, 1, 5};
    return order[e];
}

// Counting flags in LDS: wavefronts that have to meet without holding up the rest of the workgroup
// (a workgroup barrier would make the copy wavefronts wait for the query rotation and the
// computing ones for the first tile).  signal: every earlier LDS write of the wavefront is done
// first.  wait: bounded, so that a wavefront always reaches the end of the kernel.
__device__ __forceinline__ void lds_flag_signal(uint32_t* flag, int lane) {
    if (lane == 0) __hip_atomic_fetch_add(flag, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_WORKGROUP);
}
// Returns false when the count was not reached within the bound: the caller records the failed
// hand-off (the workgroup then publishes NaN partials and raises the library's fault counter)
// instead of going on silently with operands that are not there yet.
__device__ __forceinline__ bool lds_flag_wait(uint32_t* flag, uint32_t count, int spin_limit) {
    for (int spin = 0; spin < spin_limit; ++spin) {
        if (__hip_atomic_load(flag, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP) >= count) return true;
        __builtin_amdgcn_s_sleep(1);
    }
    return false;
}

// Hand-offs inside a decode workgroup that ran into their spin bound, since the library was loaded
// (read with fq_paged_decode_fault_count).
__device__ unsigned int g_decode_faults = 0u;

// Byte offset, inside a page of `H` KV heads, of chunk `cc` of the 8-head rows that head group `hgrp`
// (heads 8 hgrp .. 8 hgrp + 7) sees: the group's slices of the four sections of a token row laid end
// to end, kChunksPerRow chunks per token.  With 8 heads the slices are the row itself (16 cc).
template <bool PROD, int DIM = 128>
__device__ __forceinline__ uint32_t staged_src_offset(int cc, int H, int hgrp) {
    constexpr int CPR = StagedCfg<PROD, DIM>::CHUNKS_PER_ROW;
    const int r = cc / CPR, ci = cc - r * CPR;
    if constexpr (DIM == 256) {
        // head_dim 256, H real heads: [K idx H*128 | K norms H*4 | V idx H*128 | V norms H*4] = 264 H bytes a token;
        // group hgrp of 4 real heads
        int off;
        if (ci < 32) off = 512 * hgrp + 16 * ci;
        else if (ci == 32) off = H * 128 + 16 * hgrp;
        else if (ci < 65) off = H * 132 + 512 * hgrp + 16 * (ci - 33);
        else off = H * 260 + 16 * hgrp;
        return uint32_t(r * (H * 264) + off);
    }
    if constexpr (DIM == 64) {
        // head_dim 64, H real heads: [K idx H*32 | K norms H*4 | V idx H*32 | V norms H*4] = 72 H bytes a token
        int off;                   // group hgrp of 16 real heads
        if (ci < 32) off = 512 * hgrp + 16 * ci;
        else if (ci < 36) off = H * 32 + 64 * hgrp + 16 * (ci - 32);
        else if (ci < 68) off = H * 36 + 512 * hgrp + 16 * (ci - 36);
        else off = H * 68 + 64 * hgrp + 16 * (ci - 68);
        return uint32_t(r * (H * 72) + off);
    }
    if constexpr (PROD) {                                  // five sections: K nibbles, K norms, K residual norms, V idx, V norms
        int off;
        if (ci < 32) off = 512 * hgrp + 16 * ci;
        else if (ci < 34) off = H * 64 + 32 * hgrp + 16 * (ci - 32);
        else if (ci < 36) off = H * 68 + 32 * hgrp + 16 * (ci - 34);
        else if (ci < 68) off = H * 72 + 512 * hgrp + 16 * (ci - 36);
        else off = H * 136 + 32 * hgrp + 16 * (ci - 68);
        return uint32_t(r * (H * 140) + off);
    }
    int off;
    if (ci < 32) off = 512 * hgrp + 16 * ci;                               // K indices
    else if (ci < 34) off = H * 64 + 32 * hgrp + 16 * (ci - 32);           // K norms
    else if (ci < 66) off = H * 68 + 512 * hgrp + 16 * (ci - 34);          // V indices
    else off = H * 132 + 32 * hgrp + 16 * (ci - 66);                       // V norms
    return uint32_t(r * (H * 136) + off);
}

template <int BSL, int GP, int DT, int PVR, bool PROD, int CW, int MULTI = 0, bool STORE = false, int DIM = 128>
__global__ __launch_bounds__(512 + 64 * CW) void paged_decode_staged_kernel(const DecodeParams p) {
    constexpr bool D64 = DIM == 64, D256 = DIM == 256;
    // MULTI (0, 2, 3, 4): the kernel's rows are 1, 4, 8 or 2 consecutive tokens of 8, 2, 1 or 4 KV heads of dimension
    // 128 (1088 bytes whichever way), or, at head_dim 64, of as many pairs of heads.  Rows of several tokens (LINEAR)
    // go to LDS as they lie in the cache (with 1 and 2 heads their sections start at multiples of 4 and 8 bytes, not of
    // the 16 of a copy chunk), the computing wavefronts read their operands from where they are and merge their
    // partials at the end.
    constexpr bool LINEAR = MULTI >= 2;
    constexpr int TPR = MULTI == 4 ? 2 : 1 << MULTI;     // tokens per row
    constexpr int HPR = 8 / TPR;             // real KV heads per row
    static_assert(MULTI == 0 || (MULTI >= 2 && MULTI <= 4), "rows of 1, 2, 4 or 8 tokens");
    static_assert(!LINEAR || (!PROD && CW > 0), "rows of several tokens as they lie in the cache: TQ4, copy wavefronts");
    static_assert(!(D256 && LINEAR) || HPR % 2 == 0, "head_dim 256: the two halves of a head in one token");
    static_assert(!STORE || (CW > 0 && !PROD), "the new token is stored by the TQ4 forms with copy wavefronts");
    static_assert(DIM == 128 || (!PROD && CW > 0), "head_dim 64 / 256 are served by the TQ4 form with copy wavefronts");
    static_assert(!STORE || DIM == 128 || (DIM == 64 && LINEAR), "the new token is stored at head_dim 128, and at 64 on rows of tokens");
    // D256: the kernel's "heads" are the halves of real heads of 256 coordinates (wavefront h: real head h / 2 of the
    // group of 4, coordinates 128 (h % 2) ...): the two wavefronts of a head exchange their halves of the scores
    // through LDS every tile and add them, compute the same weights, and each accumulates its half of the output
    // coordinates.  The query comes rotated (the 256 x 256 matrix is too much for a prologue).
    // D64: the kernel's "heads" are pairs of real heads of 64 coordinates, and p.G is twice the real group size: the
    // query heads of a pair are those of its first head followed by those of its second.  A query row is the real
    // row in the half of its head and zeros in the other; its scores and outputs then are the real ones, with the
    // norms of its own head and the output coordinates of its own half.
    using Cfg = StagedCfg<PROD, DIM>;
    // LINEAR: a row of 1088 bytes every 1104 in LDS, so that the rows of a block start in eight different
    // 16-byte columns of the banks (at 1088 they would start in two)
    constexpr int kRowLds = 16 * Cfg::CHUNKS_PER_ROW + 16;    // 1104; head_dim 64: 1168
    // LINEAR: bytes of a token in such a row, and of its key (or value) norms; HPR counts heads of 128 coordinates,
    // at head_dim 64 pairs of real heads
    // or, at 256, halves of real heads
    constexpr int kTokenBytes = (D64 ? 144 : D256 ? 132 : 136) * HPR;
    constexpr int kTokenNormBytes = (D64 ? 8 : D256 ? 2 : 4) * HPR;
    constexpr int kStageBytes = LINEAR ? 16 * kRowLds : Cfg::STAGE_BYTES;
    constexpr int kTileBytes = 2 * kStageBytes;
    constexpr int kChunksPerRow = Cfg::CHUNKS_PER_ROW;
    constexpr int kChunksPerTile = Cfg::CHUNKS_PER_TILE;
    constexpr int D = 128;
    constexpr int BS = 1 << BSL;
    constexpr int KS = 4;                 // k-steps of the score product
    constexpr int DPL = 8;                // V coordinates per lane
    constexpr int NSC = GP / 2;           // scores per lane per tile
    constexpr int PPT = BS >= 32 ? 1 : 32 / BS;   // pages per tile

    // The table is a static array so that its LDS address is a compile-time constant
    // that folds into the offset field of every lookup; the tile slots are dynamic.
    __shared__ __attribute__((aligned(256))) uint32_t lut[kLutWords];
    extern __shared__ __attribute__((aligned(16))) uint8_t slots[];   // two tile slots
    // CW > 0: [0] rotated heads stored, [1] rotated (and sketched) heads read back, [2] a hand-off timed
    // out, [3 + s] tiles written to slot s (one count per copy wavefront and tile), [5 + s] tiles read
    // from slot s (one count per computing wavefront and tile)
    // STORE: [7] computing wavefronts whose part of the new token's row has reached the cache
    __shared__ uint32_t flags[8];
    // D256: [h] score halves posted by wavefront h, [8 + h] partner halves read by wavefront h (counts of tiles)
    // LINEAR: [16] computing wavefronts that have posted their partial for the merge at the end
    __shared__ uint32_t xflags[17];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int h = __builtin_amdgcn_readfirstlane(tid >> 6);   // wavefront = KV head
    bool handoff_failed = false;                             // a bounded wait of this wavefront ran out
    // CW > 0: wavefronts 8 .. 8 + CW - 1 only move tiles from the cache to LDS and the first eight
    // only consume them, so that no wavefront that computes ever waits for global memory.
    const bool copier = CW > 0 && h >= 8;
    const int n = lane & 15;
    const int g = lane >> 4;
    const int hd = n % GP;
    const int cls = n / GP;               // column class: GP=4 -> 2*block + half, GP=8 -> block, GP=16 -> 0
    // Sequence fastest: workgroups are handed to the CUs in the order of their linear index, and
    // a workgroup that finds its split empty and leaves at once does not make room for a later one
    // on another CU.  With the split index slow, the empty splits (beyond a sequence's length)
    // come last instead of alternating with the live ones.
    int seq = blockIdx.x;
    int split = blockIdx.y;
    // More than 8 KV heads: a workgroup serves the group of 8 heads blockIdx.z, i.e. the query heads
    // hq0 .. hq0 + 8 G - 1, and copies that group's slices of the token rows.
    const int hgrp = blockIdx.z;
    const int HQG = (D256 ? HPR / 2 : HPR) * p.G;        // query heads of a group
    const int hq0 = hgrp * HQG;
    const int row_bytes = D64 ? (MULTI > 0 ? 1152 : p.H_KV * 72)
                        : D256 ? (MULTI > 0 ? 1056 : p.H_KV * 264)
                               : (MULTI > 0 ? 1088 : p.H_KV * (PROD ? 140 : 136));   // a row of the cache as the kernel sees it
    const int qsub = D64 && (n % GP) >= p.G / 2 ? 1 : 0;    // D64: this lane's query head belongs to the pair's second head
    // MULTI > 0: wavefront h works on real head h % HPR and on token h / HPR of every row
    const int hh = h & (HPR - 1);                              // the kernel's head of 128 coordinates inside a token
    const int hr = D256 ? (hh >> 1) : hh;                      // D256: the real head; its half is h & 1
    const int tsel = (h / HPR) & (TPR - 1);

    // Every load that depends on nothing is asked for first, so that the memory
    // latencies of the prologue overlap instead of adding up: the centroids, the
    // rotation columns of this wavefront and the first 32 query heads.
    // K table in the lower 128 bytes of every 256-byte table row (32 copies, one per bank),
    // V table in the upper 128 bytes
    const float cent_k_mine = p.centroids_k[lane & (PROD ? 7 : 15)];
    const float cent_v_mine = p.centroids_v[lane & 15];
    const uint8_t* lut_k = reinterpret_cast<const uint8_t*>(lut);
    const uint8_t* lut_v = lut_k;
    const uint32_t lane_off = 4u * (lane & 31);
    const uint32_t lane_off_v = 128u + lane_off;
    float rot_b[4][8];
    float rot_s[4][8];
    auto load_matrix_columns = [&]() {
        if (p.rotation != nullptr && !copier) {
            if constexpr (D64) {
                // the 64 x 64 matrix twice on the diagonal of the 128 x 128 one: wavefront h has columns 16 h .. 16 h + 15
                float b64[2][8];
                load_rotation_any<64>(p.rotation, p.rot_col_major != 0, true, 16 * (h & 3), n, g, b64);
#pragma unroll
                for (int j = 0; j < 4; ++j)
#pragma unroll
                    for (int e = 0; e < 8; ++e) rot_b[j][e] = (j >> 1) == (h >> 2) ? b64[j & 1][e] : 0.0f;
            } else {
                load_rotation_any<128>(p.rotation, p.rot_col_major != 0, true, 16 * h, n, g, rot_b);
            }
            if constexpr (PROD) load_rotation_any<128>(p.sketch, false, true, 16 * h, n, g, rot_s);
        }
    };
    // With copy wavefronts the sequence length and the page ids are asked for first (below): the
    // first tile hangs on them, the query rotation has time.
    if constexpr (CW == 0) load_matrix_columns();

    // Everything that depends on the lane alone is worked out here, while the first loads are on
    // their way: the first value that comes back from memory is needed 2.5 us after entry.
    // ---- copy plan: chunk c = tid + 512 k of the tile, k = 0..3; the remaining chunks go out as
    // one dword per thread where that comes out even (128 chunks = 512 dwords: every wavefront
    // then moves the same amount), else as whole chunks by the first wavefronts ------------------
    constexpr int ROUNDS = 5;
    constexpr bool kSpreadTail = (kChunksPerTile - 4 * 512) * 4 == 512;
    uint32_t src_off[ROUNDS];    // byte offset from the base of the chunk's page
    int src_page[ROUNDS];        // which of the tile's pages (lane constant)
    int dst_off[ROUNDS];         // byte offset inside the LDS tile slot
#pragma unroll
    for (int k = 0; k < ROUNDS; ++k) {
        if constexpr (CW > 0) {   // the copy wavefronts have a plan of their own
            src_off[k] = 0u;
            src_page[k] = 0;
            dst_off[k] = 0;
            continue;
        }
        int c = (tid & 511) + 512 * k;
        if (kSpreadTail && k == 4) c = 4 * 512 + ((tid & 511) >> 2);
        c = c < kChunksPerTile ? c : kChunksPerTile - 1;
        // rows of a page are contiguous: chunk c of the tile is chunk c - page * (chunks per page) of its page
        constexpr int PC = BS * kChunksPerRow;
        int pg = 0;
#pragma unroll
        for (int i = 1; i < PPT; ++i) pg += c >= i * PC ? 1 : 0;
        src_page[k] = pg;
        const int sub = (kSpreadTail && k == 4) ? 4 * (tid & 3) : 0;
        src_off[k] = staged_src_offset<PROD, DIM>(c - pg * PC, p.H_KV, hgrp) + uint32_t(sub);
        dst_off[k] = kChunkDst<PROD, DIM>.off[c] + sub;
    }
    const bool has_round4 = kSpreadTail || tid < kChunksPerTile - 4 * 512;   // else whole wavefronts
    // ---- lane-constant LDS read offsets (inside a tile slot) -------------------------------
    int k_rd[2];                // K operand of block b: 16 bytes of row n, quarter g
    int v_rd[2][4];             // V operand: dword n of rows 4g + i of block b
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        if constexpr (LINEAR) {
            // the token rows as they lie in the cache: token tsel of the row, head hr of its HPR heads
            const int token = kTokenBytes * tsel;
            k_rd[b] = b * kStageBytes + kRowLds * n + token + 64 * hh + 16 * g;
#pragma unroll
            for (int i = 0; i < 4; ++i)
                v_rd[b][i] = b * kStageBytes + kRowLds * (4 * g + i) + token + 64 * HPR + kTokenNormBytes + 64 * hh + 4 * n;
        } else {
            k_rd[b] = b * kStageBytes + 16 * staged_slot(h, n, g);
#pragma unroll
            for (int i = 0; i < 4; ++i)
                v_rd[b][i] = b * kStageBytes + 8192 + 16 * staged_slot(h, 4 * g + i, n >> 2) + 4 * (n & 3);
        }
    }
    // the (block, row) of this lane's scores, and the slot of each score in the P operand
    int sc_tok[NSC];            // token offset inside the tile
    int n_rd[NSC];              // K norm offset; the V norm is 512 bytes further (LINEAR: the V indices and K norms of the token's heads)
#pragma unroll
    for (int e = 0; e < NSC; ++e) {
        int blk, row;
        if (GP == 4) { blk = cls >> 1; row = 4 * g + 2 * (cls & 1) + e; }
        else if (GP == 8) { blk = cls; row = 4 * g + e; }
        else { blk = e >> 2; row = 4 * g + (e & 3); }
        sc_tok[e] = 16 * blk + row;
        n_rd[e] = LINEAR ? blk * kStageBytes + kRowLds * row + kTokenBytes * tsel + 64 * HPR + (D64 ? 8 * hr + 4 * qsub : 4 * hr)
                : D64 ? blk * kStageBytes + Cfg::KN_OFF + 64 * row + 8 * h + 4 * qsub
                : D256 ? blk * kStageBytes + Cfg::KN_OFF + 16 * row + 4 * (h >> 1)
                       : blk * kStageBytes + kStageKnOff + 32 * row + 4 * h;
    }

    // dword d of the P operand holds slots 2d, 2d + 1: it is this lane's when its class owns them
    uint32_t pa_mask[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        bool mine;
        if (GP == 4) mine = d == cls;                 // class = 2 * block + half, one dword each
        else if (GP == 8) mine = (d >> 1) == cls;     // class = block, two dwords each
        else mine = true;
        pa_mask[d] = mine ? 0xffffffffu : 0u;
    }

    __builtin_amdgcn_sched_barrier(0);
    const int NS = p.num_splits;
    const bool rowwide = p.max_blocks <= 64 * PVR;
    // every sequence is cut into the same token chunks (those of the longest possible context):
    // the work of a workgroup does not depend on its sequence's length, short sequences just
    // leave their last splits empty
    int chunk = (((p.max_blocks * BS + NS - 1) / NS) + 63) & ~63;
    int L_known = -1;
    if (p.balance_slots > 0) balance_chunks<PVR, BS, TPR>(p, lane, NS, rowwide, chunk, seq, split, L_known);

    const uint16_t* qseq = reinterpret_cast<const uint16_t*>(p.q_rot) + (int64_t(seq) * p.H_Q + hq0) * DIM;
    // eight elements of query row `row` of this workgroup, from element `v` (a multiple of 8) of the 128 the kernel
    // works on.  D64: the real row of 64 in the half of its head, zeros in the other half.
    auto q_chunk = [&](int row, int v) -> uint4v {
        if constexpr (D256) {
            return *reinterpret_cast<const uint4v*>(qseq + row * 256 + 128 * (h & 1) + v);     // this wavefront's half
        } else if constexpr (!D64) {
            return *reinterpret_cast<const uint4v*>(qseq + row * 128 + v);
        } else {
            const int in_group = row - (row / p.G) * p.G;
            const int row_sub = in_group >= p.G / 2 ? 1 : 0;
            const uint4v x = *reinterpret_cast<const uint4v*>(qseq + row * 64 + (v & 63));
            return (v >> 6) == row_sub ? x : uint4v{0u, 0u, 0u, 0u};
        }
    };
    uint4v q_pre[2][4];
    auto load_first_heads = [&]() {
        if (p.rotation != nullptr && !copier) {
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                const int row = 16 * rb + n < HQG ? 16 * rb + n : HQG - 1;
#pragma unroll
                for (int j = 0; j < 4; ++j) q_pre[rb][j] = q_chunk(row, 32 * j + 8 * g);
            }
        }
    };
    if constexpr (CW == 0) load_first_heads();
    // Page ids.  When the whole block-table row fits the registers (64 * PVR pages) it is
    // fetched now, before the sequence length is known, so that the two loads overlap;
    // otherwise the registers hold the pages of this split, which depend on the length.
    const int32_t* bt = p.block_table + int64_t(seq) * p.max_blocks;
    int pv[PVR];
#pragma unroll
    for (int r = 0; r < PVR; ++r) pv[r] = 0;
    const bool copies = CW == 0 || copier;   // this wavefront moves tiles: it needs the page ids
    if (rowwide && copies) {
#pragma unroll
        for (int r = 0; r < PVR; ++r) {
            const int idx = 64 * r + lane < p.max_blocks ? 64 * r + lane : p.max_blocks - 1;
            pv[r] = bt[idx];
        }
    }

    int L = L_known;
    if (L_known < 0) L = p.seq_lens[seq];
    if constexpr (CW > 0) {
        // The flags are cleared behind a barrier placed where nobody waits for anybody: every
        // wavefront has just asked for its sequence length and page ids and none has used them yet
        // (the barrier does not wait for loads from global memory).
        if (tid < 8) flags[tid] = 0u;
        if ((D256 || LINEAR) && tid < 17) xflags[tid] = 0u;
        __syncthreads();
        load_matrix_columns();
        load_first_heads();
    }
    // STORE: the new token's rows and slot are asked for with the other prologue loads, by every workgroup
    // (which one needs them depends on the sequence length, which is on its way)
    constexpr int kNewHeads = HPR;                          // KV heads of this workgroup
    uint4v new_raw[4];
    int64_t new_slot = -1;
    float bnd_mine = 0.0f;      // boundary `lane` of the 15 (asked for here: at its use it would be a round trip of its own)
    if constexpr (STORE) {
        if (!copier) {
            const int kv_heads = MULTI > 0 ? HPR : p.H_KV;       // (head_dim 64: pairs of heads, 128 elements together)
            const int nr = n < 2 * kNewHeads ? n : 2 * kNewHeads - 1;     // block row: key head nr, or value head nr - KH
            const uint16_t* xrow = reinterpret_cast<const uint16_t*>(nr < kNewHeads ? p.new_key : p.new_value) +
                                   (int64_t(seq) * kv_heads + kNewHeads * hgrp + (nr & (kNewHeads - 1))) * 128;
#pragma unroll
            for (int j = 0; j < 4; ++j) new_raw[j] = *reinterpret_cast<const uint4v*>(xrow + 32 * j + 8 * g);
            new_slot = p.new_slots[seq];
            bnd_mine = p.boundaries[lane < 15 ? lane : 14];
        }
    }
    L = L < 0 ? 0 : L;
    L = L > p.max_blocks * BS * TPR ? p.max_blocks * BS * TPR : L;
    // MULTI > 0: from here on L counts rows (of TPR tokens); the last row may hold no token of this wavefront
    const int rows_mine = (L + TPR - 1 - tsel) / TPR;
    L = (L + TPR - 1) / TPR;
    const int begin = split * chunk;
    const int end = L < begin + chunk ? L : begin + chunk;
    const int end_mine = rows_mine < end ? rows_mine : end;      // rows < end_mine hold a token of this wavefront
    const int hq_lane = hr * p.G + n;
    // (rows of several tokens: the wavefronts of a head merge their partials into the one of the split)
    const int NS_out = NS;
    const int split_out = split;
    if (begin >= end) {   // uniform over the workgroup
        if (g == 0 && n < p.G && !copier && (!D256 || (h & 1) == 0) && (!LINEAR || tsel == 0)) {
            const int64_t o = (int64_t(seq) * p.H_Q + hq0 + hq_lane) * NS_out + split_out;
            p.part_m[o] = -__builtin_inff();
            p.part_l[o] = 0.0f;
        }
        return;
    }
    const int last_page_idx = (L - 1) >> BSL;
    const int max_page = p.num_blocks - 1;
    const uint8_t* cache = p.cache;
    const int64_t page_bytes = int64_t(BS) * row_bytes;

    // ---- page ids of the split in registers (see the direct kernel) ---------------------
    const int split_p0 = rowwide ? 0 : begin >> BSL;   // page index held by lane 0 of pv[0]
    if (!rowwide && copies) {
#pragma unroll
        for (int r = 0; r < PVR; ++r) {
            int idx = split_p0 + 64 * r + lane;
            idx = idx > last_page_idx ? last_page_idx : idx;
            pv[r] = bt[idx];
        }
    }
    auto page_id = [&](int rel) -> int {
        int v = __builtin_amdgcn_readlane(pv[0], rel & 63);
#pragma unroll
        for (int r = 1; r < PVR; ++r) {
            const int vr = __builtin_amdgcn_readlane(pv[r], rel & 63);
            v = (rel >> 6) == r ? vr : v;
        }
        return v;
    };
    // the table is filled while the page ids are on their way
    if (!copier) fill_pair_tables<8>(lut, cent_k_mine, cent_v_mine, PROD ? 7 : 15, h, lane);


    uint4v stage_reg[ROUNDS];
    auto issue_loads = [&](int t0) {
        const uint8_t* base[PPT];
        const int p0 = (t0 >> BSL) - split_p0;
#pragma unroll
        for (int i = 0; i < PPT; ++i) base[i] = cache + int64_t(page_id(p0 + i)) * page_bytes;
        const uint32_t in_page = BS >= 32 ? uint32_t((t0 & (BS - 1)) * row_bytes) : 0u;
#pragma unroll
        for (int k = 0; k < ROUNDS; ++k) {
            // where a page is a whole number of wavefront rounds (16 rows of 68 chunks = 17 x 64), a
            // wavefront's 64 chunks lie in one page and the page base stays in scalar registers
            constexpr bool kUniformPage = (BS * kChunksPerRow) % 64 == 0;
            const int pg_k = kUniformPage ? __builtin_amdgcn_readfirstlane(src_page[k]) : src_page[k];
            const uint8_t* b = base[0];
#pragma unroll
            for (int i = 1; i < PPT; ++i) b = pg_k == i ? base[i] : b;
            if (kSpreadTail && k == 4) stage_reg[k].x = *reinterpret_cast<const uint32_t*>(b + in_page + src_off[k]);
            else if (k < 4 || has_round4) stage_reg[k] = *reinterpret_cast<const uint4v*>(b + in_page + src_off[k]);
        }
    };
    auto write_slot = [&](int slot) {
        uint8_t* dst = slots + slot * kTileBytes;
#pragma unroll
        for (int k = 0; k < ROUNDS; ++k)
            if (kSpreadTail && k == 4) *reinterpret_cast<uint32_t*>(dst + dst_off[k]) = stage_reg[k].x;
            else if (k < 4 || has_round4) *reinterpret_cast<uint4v*>(dst + dst_off[k]) = stage_reg[k];
    };

#pragma unroll
    for (int r = 0; r < PVR; ++r) pv[r] = pv[r] < 0 ? 0 : (pv[r] > max_page ? max_page : pv[r]);
    const int last_t0 = begin + ((end - begin - 1) & ~31);
    auto clamp_t0 = [&](int t) { return t < last_t0 ? t : last_t0; };
    // STORE: this workgroup's split ends with the sequence's last token, the one this step adds: its
    // computing wavefronts write that token's cache row in the prologue, and its copy wavefronts ask
    // for the split's last tile only after that (uniform over the workgroup)
    const bool stores_token = STORE && end == L;

    if constexpr (CW > 0) {
        if (copier) {
            // ---- the copy wavefronts: chunk c = ct + 64 CW k of a tile, the rest as 8 bytes per
            // thread; two tiles in flight in registers (sets A and B), each written to the slot that
            // the tile two before it has just left --------------------------------------------------
            constexpr int CT = 64 * CW;
            constexpr int FULL = kChunksPerTile / CT;
            constexpr int REST = kChunksPerTile - FULL * CT;
            constexpr bool kHalfTail = REST * 2 == CT;   // else whole chunks by the first REST threads
            constexpr int NR = REST > 0 ? FULL + 1 : FULL;   // register sets of a tile: the whole rounds and the rest
            const int ct = tid - 512;
            uint32_t c_src[NR];
            int c_page[NR];
            int c_dst[NR];
#pragma unroll
            for (int k = 0; k < NR; ++k) {
                int c = k < FULL ? ct + CT * k : FULL * CT + (kHalfTail ? ct >> 1 : ct);
                c = c < kChunksPerTile ? c : kChunksPerTile - 1;
                constexpr int PC = BS * kChunksPerRow;
                int pg = 0;
#pragma unroll
                for (int i = 1; i < PPT; ++i) pg += c >= i * PC ? 1 : 0;
                c_page[k] = pg;
                const int sub = (k < FULL || !kHalfTail) ? 0 : 8 * (ct & 1);
                if constexpr (LINEAR) {     // the rows of a page, and of a tile in LDS, one after the other
                    c_src[k] = 16u * uint32_t(c - pg * PC) + uint32_t(sub);
                    c_dst[k] = kRowLds * (c / kChunksPerRow) + 16 * (c % kChunksPerRow) + sub;
                } else {
                    c_src[k] = staged_src_offset<PROD, DIM>(c - pg * PC, p.H_KV, hgrp) + uint32_t(sub);
                    c_dst[k] = kChunkDst<PROD, DIM>.off[c] + sub;
                }
            }
            const bool has_rest = kHalfTail || ct < REST;
            auto c_issue = [&](uint4v (&r)[NR], int t0) {
                if (t0 > last_t0) return;             // beyond the split: nothing to fetch
                if constexpr (STORE) {
                    if (stores_token && t0 == last_t0 && !lds_flag_wait(&flags[7], 8u, p.spin_limit)) flags[2] = 1u;
                }
                constexpr int NBASE = LINEAR ? 1 : PPT;
                const uint8_t* base[NBASE];
                const int p0 = (t0 >> BSL) - split_p0;
                if constexpr (!LINEAR) {
#pragma unroll
                    for (int i = 0; i < PPT; ++i) base[i] = cache + int64_t(page_id(p0 + i)) * page_bytes;
                }
                const uint32_t in_page = BS >= 32 ? uint32_t((t0 & (BS - 1)) * row_bytes) : 0u;
                // LINEAR: a tile has 4 to 16 pages and a lane's chunks lie in several of them.  The tile's first page
                // index is a multiple of its page count, so all its pages sit in one of the page-id registers, and
                // a lane fetches the id of each of its pages from the lane that holds it.
                int pv_tile = pv[0];
                if constexpr (LINEAR) {     // (masks, not selects: the compiler turns a chain of selects on pv[] into
                                            // an indexed array in scratch memory)
                    const int sel = __builtin_amdgcn_readfirstlane(p0 >> 6);
                    pv_tile = 0;
#pragma unroll
                    for (int r = 0; r < PVR; ++r) pv_tile |= pv[r] & (sel == r ? -1 : 0);
                }
#pragma unroll
                for (int k = 0; k < NR; ++k) {
                    const uint8_t* b;
                    if constexpr (LINEAR) {
                        const int id = __builtin_amdgcn_ds_bpermute(4 * ((p0 & 63) + c_page[k]), pv_tile);
                        b = cache + int64_t(id) * page_bytes;
                    } else {
                        constexpr bool kUniformPage = (BS * kChunksPerRow) % 64 == 0;
                        const int pg_k = kUniformPage ? __builtin_amdgcn_readfirstlane(c_page[k]) : c_page[k];
                        b = base[0];
#pragma unroll
                        for (int i = 1; i < PPT; ++i) b = pg_k == i ? base[i] : b;
                    }
                    if (k < FULL) {
                        r[k] = *reinterpret_cast<const uint4v*>(b + in_page + c_src[k]);
                    } else if (!kHalfTail) {
                        if (has_rest) r[k] = *reinterpret_cast<const uint4v*>(b + in_page + c_src[k]);
                    } else {
                        const uint2v t = *reinterpret_cast<const uint2v*>(b + in_page + c_src[k]);
                        r[k].x = t.x;
                        r[k].y = t.y;
                    }
                }
            };
            auto c_write = [&](int slot, const uint4v (&r)[NR]) {
                uint8_t* dst = slots + slot * kTileBytes;
#pragma unroll
                for (int k = 0; k < NR; ++k) {
                    if (k < FULL) *reinterpret_cast<uint4v*>(dst + c_dst[k]) = r[k];
                    else if (!kHalfTail) { if (has_rest) *reinterpret_cast<uint4v*>(dst + c_dst[k]) = r[k]; }
                    else *reinterpret_cast<uint2v*>(dst + c_dst[k]) = uint2v{r[k].x, r[k].y};
                }
            };
            uint4v ra[NR], rb[NR];
#pragma unroll
            for (int k = 0; k < NR; ++k) ra[k] = rb[k] = uint4v{0u, 0u, 0u, 0u};
            c_issue(ra, begin);
            c_issue(rb, begin + 32);
            // Producer side of a bounded buffer of two LDS slots, synchronised with counting flags
            // instead of workgroup barriers: the copy and the computing wavefronts are not in step
            // with each other, nor the computing wavefronts among themselves.  Tile j goes to slot
            // j % 2, which last held tile j - 2: it is free when all eight computing wavefronts have
            // read j / 2 tiles from it (none can be further: tile j is not there yet).  The query
            // exchange of the computing wavefronts goes through the second slot and, with a sketch,
            // the first: the first write to those waits until all eight have read their heads back.
            int j = 0;
            for (int t0 = begin; t0 < end; t0 += 32, ++j) {
                if (j >= 2 && !lds_flag_wait(&flags[5 + (j & 1)], 8u * uint32_t(j >> 1), p.spin_limit)) flags[2] = 1u;
                if (p.rotation != nullptr && j == (PROD ? 0 : 1) && !lds_flag_wait(&flags[1], 8u, p.spin_limit)) flags[2] = 1u;
                if (j & 1) {
                    c_write(1, rb);
                    lds_flag_signal(&flags[4], lane);
                    c_issue(rb, t0 + 64);
                } else {
                    c_write(0, ra);
                    lds_flag_signal(&flags[3], lane);
                    c_issue(ra, t0 + 64);
                }
            }
            return;
        }
    }
    // the loads of the first tile fly while the query is prepared
    if constexpr (CW == 0) issue_loads(begin);

    // ---- query operand ------------------------------------------------------------------
    // With a rotation matrix the workgroup first rotates all query heads of its sequence:
    // wavefront h produces columns 16h .. 16h+15 of q_rot = (q @ R.T) on the float32 MFMA,
    // rounded to the query dtype as the reference rounds it, and the heads are exchanged
    // through LDS (the tile slots are not in use yet).
    half8 qh[KS];
    half8 qsh[KS];              // PROD: sketched query S q (times sqrt(pi/2) / D), elements in sign order
    float qscale;
    float qscale_s = 0.0f;
    {
        float qf[KS][8];
        float mx = 0.0f;
        const bool live = hd < p.G;
        if (p.rotation != nullptr) {
            // The rotated heads are exchanged through the second tile slot as 16-bit words of the
            // query dtype (32 KB for 128 heads): the first tile goes to the first slot, and the
            // second slot is not written before the barrier of the first loop iteration, which
            // every wavefront reaches after it has read its heads back.  With a sketch the
            // float32 sketched query (H_Q <= 64) takes the first slot and a barrier of its own.
            uint16_t* qs = reinterpret_cast<uint16_t*>(slots + kTileBytes);
            float* qs2 = reinterpret_cast<float*>(slots);
            // This wavefront's 16 matrix columns.  bfloat16 heads go to the bf16 MFMA as loaded, against
            // the columns in three bf16 terms; fp16 heads are scaled by a power of two and go to the fp16
            // MFMA against two fp16 terms.  Either way the products are exact.
            constexpr bool kRawBf16 = DT == FQ_BF16;
            half8 rot_hi[KS], rot_lo[KS], sk_hi[KS], sk_lo[KS];
            bf16v8 rot_t[3][KS], sk_t[3][KS];
            if constexpr (kRawBf16) {
                split_rotation_block_bf16<D>(rot_b, rot_t);
                if constexpr (PROD) split_rotation_block_bf16<D>(rot_s, sk_t);
            } else {
                split_rotation_block<D>(rot_b, rot_hi, rot_lo);
                if constexpr (PROD) split_rotation_block<D>(rot_s, sk_hi, sk_lo);
            }
            for (int rb = 0; 16 * rb < HQG; ++rb) {
                const int row = 16 * rb + n < HQG ? 16 * rb + n : HQG - 1;
                uint4v raw[KS];
#pragma unroll
                for (int j = 0; j < KS; ++j)
                    raw[j] = rb < 2 ? q_pre[rb & 1][j] : q_chunk(row, 32 * j + 8 * g);
                float4v acc, acc2 = {0.f, 0.f, 0.f, 0.f};
                float up = 1.0f;
                if constexpr (kRawBf16) {
                    bf16v8 a[KS];
#pragma unroll
                    for (int j = 0; j < KS; ++j) a[j] = __builtin_bit_cast(bf16v8, raw[j]);
                    acc = rotate_block_bf16<D>(a, rot_t);
                    if constexpr (PROD) acc2 = rotate_block_bf16<D>(a, sk_t);
                } else {
                    half8 a[KS];
                    rows_as_f16<D, DT>(raw, a, up);
                    acc = rotate_block_f16<D>(a, rot_hi, rot_lo);
                    if constexpr (PROD) acc2 = rotate_block_f16<D>(a, sk_hi, sk_lo);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int head = 16 * rb + 4 * g + i;
                    if (head < HQG) qs[head * D + 16 * h + n] = store_elem<DT>(acc[i] * up);
                }
                if constexpr (PROD) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int head = 16 * rb + 4 * g + i;
                        if (head < HQG) qs2[head * D + 16 * h + n] = acc2[i] * up;
                    }
                }
            }
            if constexpr (STORE) {
                if (stores_token) {
                    // ---- the new token: TQ4 compress of its key and value rows (KH of each: one more block of
                    // 16 rows for the same matrix product) straight into the cache row: n = ||x||,
                    // y = (x R^T) / (n + 1e-10), index = number of boundaries below y, two indices per byte
                    // (cpu_reference.py:22-61, vllm/impl.py:220-263).  Wavefront h holds columns 16h..16h+15.
                    // Block row r: key head r for r < KH, value head r - KH for r < 2 KH.
                    constexpr int KH = kNewHeads;
                    const int token_row_bytes = MULTI > 0 ? kTokenBytes : row_bytes;
                    const int kv_heads = MULTI > 0 ? HPR : p.H_KV;
                    const int64_t slot = new_slot;
                    uint4v raw[KS];
#pragma unroll
                    for (int j = 0; j < KS; ++j) raw[j] = new_raw[j];
                    // sum of squares of row n: this lane's 32 elements, then over g.  head_dim 64: a row is a pair of heads,
                    // elements 0..63 the first and 64..127 the second; wavefront h holds columns of head h / 4 of the pair
                    float ss = 0.0f;
#pragma unroll
                    for (int j = 0; j < KS; ++j) {
                        const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
                        const bool mine = !D64 || (j >> 1) == (h >> 2);
#pragma unroll
                        for (int i = 0; i < 4; ++i) {
                            const float a = load_elem<DT>(uint16_t(w[i] & 0xffffu)), b = load_elem<DT>(uint16_t(w[i] >> 16));
                            ss = mine ? __builtin_fmaf(a, a, ss) : ss;
                            ss = mine ? __builtin_fmaf(b, b, ss) : ss;
                        }
                    }
                    ss += xor_shuffle(ss, 16);
                    ss += xor_shuffle(ss, 32);
                    float4v acc;
                    float up = 1.0f;
                    if constexpr (kRawBf16) {
                        bf16v8 a[KS];
#pragma unroll
                        for (int j = 0; j < KS; ++j) a[j] = __builtin_bit_cast(bf16v8, raw[j]);
                        acc = rotate_block_bf16<D>(a, rot_t);
                    } else {
                        half8 a[KS];
                        rows_as_f16<D, DT>(raw, a, up);
                        acc = rotate_block_f16<D>(a, rot_hi, rot_lo);
                    }
                    const bool stored = slot >= 0 && slot < p.num_slots;
                    uint8_t* crow = p.cache_rw + (stored ? slot : 0) * int64_t(token_row_bytes);
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const int r = 4 * g + i;                     // row of the block
                        const float ssr = __shfl(ss, r, kWave);
                        const bool tiny = ssr < 0x1p-96f;            // as the compress kernel: v_sqrt_f32 on a normal number
                        const float nrm_s = __builtin_amdgcn_sqrtf(tiny ? ssr * 0x1p64f : ssr);
                        const float nrm = tiny ? nrm_s * 0x1p-32f : nrm_s;
                        const float y = acc[i] * (up * __builtin_amdgcn_rcpf(nrm + 1e-10f));
                        uint32_t idx = 0u;
#pragma unroll
                        for (int k = 0; k < 15; ++k)
                            idx += bits_to_float(uint32_t(__builtin_amdgcn_readlane(int(float_to_bits(bnd_mine)), k))) < y ? 1u : 0u;
                        // byte j of a head = index of coordinate 2j (high nibble) and 2j + 1: columns n, n + 1
                        const uint32_t other = uint32_t(__shfl_xor(int(idx), 1, kWave));
                        const uint32_t byte = (idx << 4) | other;                        // valid in even n
                        uint32_t lo = (n & 9) == 0 ? byte << (4 * (n & 6)) : 0u;         // n = 0, 2, 4, 6: bytes 0..3
                        uint32_t hi = (n & 9) == 8 ? byte << (4 * (n & 6)) : 0u;         // n = 8 .. 14: bytes 4..7
#pragma unroll
                        for (int mask = 2; mask < 16; mask <<= 1) {
                            lo |= uint32_t(__shfl_xor(int(lo), mask, kWave));
                            hi |= uint32_t(__shfl_xor(int(hi), mask, kWave));
                        }
                        const int head = KH * hgrp + (r & (KH - 1));
                        const int sect = r < KH ? 0 : kv_heads * (D / 2 + (D64 ? 8 : 4));   // key sections, then value sections
                        const bool row_live = stored && r < 2 * KH;
                        if (row_live && n == 0)
                            *reinterpret_cast<uint2v*>(crow + sect + head * (D / 2) + 8 * h) = uint2v{lo, hi};
                        if constexpr (D64) {     // two norms a pair: wavefronts 0 and 4 hold those of its first and second head
                            if (row_live && n == 1 && (h & 3) == 0)
                                *reinterpret_cast<float*>(crow + sect + kv_heads * (D / 2) + 8 * head + 4 * (h >> 2)) = nrm;
                        } else {
                            if (row_live && n == 1 && h == 0)
                                *reinterpret_cast<float*>(crow + sect + kv_heads * (D / 2) + 4 * head) = nrm;
                        }
                    }
                    // The row must be in the cache before the copy wavefronts ask for the split's last tile.  They
                    // ask for the first two tiles at once; when the last tile is one of those the stores are waited
                    // for here, otherwise after the first tile's arithmetic, when they have long completed.
                    if (last_t0 < begin + 64) {
                        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                        lds_flag_signal(&flags[7], lane);
                    }
                }
            }
            if constexpr (CW > 0) {
                lds_flag_signal(&flags[0], lane);
                if (!lds_flag_wait(&flags[0], 8u, p.spin_limit)) { flags[2] = 1u; handoff_failed = true; }
            } else {
                __syncthreads();
            }
            const uint16_t* src = qs + (hr * p.G + (live ? hd : 0)) * D + g * (D / 4);
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint4v raw = *reinterpret_cast<const uint4v*>(src + 8 * ks);
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    qf[ks][2 * i] = live ? load_elem<DT>(uint16_t(w[i] & 0xffffu)) : 0.0f;
                    qf[ks][2 * i + 1] = live ? load_elem<DT>(uint16_t(w[i] >> 16)) : 0.0f;
                    mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(qf[ks][2 * i]), __builtin_fabsf(qf[ks][2 * i + 1])));
                }
            }
            if constexpr (PROD) {
                // <S q, signs> * sqrt(pi/2) / D: the constant rides on the query side
                const float* src2 = qs2 + (hr * p.G + (live ? hd : 0)) * D + g * (D / 4);
                float qf2[KS][8];
                float mx2 = 0.0f;
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        qf2[ks][e] = live ? src2[8 * ks + sign_order(e)] * (1.2533141373155003f / float(D)) : 0.0f;
                        mx2 = __builtin_fmaxf(mx2, __builtin_fabsf(qf2[ks][e]));
                    }
                mx2 = max_xor32(max_xor16(mx2));
                int ex2 = int((float_to_bits(mx2) >> 23) & 0xffu) - 127;
                if (ex2 < -100 || ex2 > 100) ex2 = 0;
                const float down2 = bits_to_float(uint32_t(127 - ex2) << 23);
                qscale_s = p.scale_log2e * bits_to_float(uint32_t(127 + ex2) << 23);
#pragma unroll
                for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                    for (int e = 0; e < 8; ++e) qsh[ks][e] = _Float16(qf2[ks][e] * down2);
            }
            // the heads are read back: the slots they went through may receive tiles
            if constexpr (CW > 0) lds_flag_signal(&flags[1], lane);
            else if constexpr (PROD) __syncthreads();
        } else {
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const uint4v raw = q_chunk(hr * p.G + (live ? hd : 0), g * (D / 4) + 8 * ks);
                const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    qf[ks][2 * i] = live ? load_elem<DT>(uint16_t(w[i] & 0xffffu)) : 0.0f;
                    qf[ks][2 * i + 1] = live ? load_elem<DT>(uint16_t(w[i] >> 16)) : 0.0f;
                    mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(qf[ks][2 * i]), __builtin_fabsf(qf[ks][2 * i + 1])));
                }
            }
        }
        mx = max_xor32(max_xor16(mx));
        int ex = int((float_to_bits(mx) >> 23) & 0xffu) - 127;
        if (ex < -100 || ex > 100) ex = 0;
        const float down = bits_to_float(uint32_t(127 - ex) << 23);
        qscale = p.scale_log2e * bits_to_float(uint32_t(127 + ex) << 23);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) qh[ks][e] = _Float16(qf[ks][e] * down);
    }

    // ---- running state ---------------------------------------------------------------------
    float4v O[DPL];
#pragma unroll
    for (int db = 0; db < DPL; ++db) O[db] = float4v{0.f, 0.f, 0.f, 0.f};
    float M = -__builtin_inff();
    float lsum = 0.0f;

    auto compute_tile = [&](int t0, int slot, int it) {
        const uint8_t* tile = slots + slot * kTileBytes;
        // operands of this lane, raw
        uint4v kraw[2];
        uint32_t vraw[2][4];
        float kn[NSC], vn[NSC], kg[NSC];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            if constexpr (LINEAR) {     // a token's index bytes start at a multiple of 8 bytes
                const uint2v lo = *reinterpret_cast<const uint2v*>(tile + k_rd[b]);
                const uint2v hi = *reinterpret_cast<const uint2v*>(tile + k_rd[b] + 8);
                kraw[b] = uint4v{lo.x, lo.y, hi.x, hi.y};
            } else {
                kraw[b] = *reinterpret_cast<const uint4v*>(tile + k_rd[b]);
            }
        }
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int i = 0; i < 4; ++i) vraw[b][i] = *reinterpret_cast<const uint32_t*>(tile + v_rd[b][i]);
#pragma unroll
        for (int e = 0; e < NSC; ++e) {
            kn[e] = *reinterpret_cast<const float*>(tile + n_rd[e]);
            vn[e] = *reinterpret_cast<const float*>(tile + n_rd[e] + (LINEAR ? 64 * HPR + kTokenNormBytes : DIM != 128 ? Cfg::VN_OFF - Cfg::KN_OFF : kStageVnOff - kStageKnOff));
            kg[e] = PROD ? *reinterpret_cast<const float*>(tile + n_rd[e] + (kStageKgOff - kStageKnOff)) : 0.0f;
        }
        // These were all the reads of the slot (the lookups below go to the table): it is handed back
        // to the copy wavefronts here, long before the tile's arithmetic is done (the release waits
        // for the reads to complete).
        if constexpr (CW > 0) lds_flag_signal(&flags[5 + slot], lane);

        // ---- scores: lookups of block 1 in flight during the MFMAs of block 0 ----------------
        uint4v ka[2][KS];
        const uint32_t kw[2][4] = {{kraw[0].x, kraw[0].y, kraw[0].z, kraw[0].w}, {kraw[1].x, kraw[1].y, kraw[1].z, kraw[1].w}};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) ka[0][ks] = lookup_word(lut_k, kw[0][ks], lane_off);
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) ka[1][ks] = lookup_word(lut_k, kw[1][ks], lane_off);
        // nibble transposes of the V token pairs: pair jp = rows (2 jp', 2 jp' + 1) of block jp / 2
        uint32_t X[4], Y[4];
#pragma unroll
        for (int jp = 0; jp < 4; ++jp) {
            const uint32_t A = vraw[jp >> 1][2 * (jp & 1)], B = vraw[jp >> 1][2 * (jp & 1) + 1];
            X[jp] = (A & 0xF0F0F0F0u) | ((B >> 4) & 0x0F0F0F0Fu);
            Y[jp] = ((A << 4) & 0xF0F0F0F0u) | (B & 0x0F0F0F0Fu);
        }
        uint4v vb[2][4];
        auto v_group = [&](int grp, uint4v (&dst)[4]) {   // coordinate blocks 4 grp .. 4 grp + 3
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int db = 4 * grp + e, bi = db / 2;
                const uint32_t (&src)[4] = (db & 1) ? Y : X;
                dst[e] = (bi == 0) ? lookup_column<0>(lut_v, src, lane_off_v)
                       : (bi == 1) ? lookup_column<1>(lut_v, src, lane_off_v)
                       : (bi == 2) ? lookup_column<2>(lut_v, src, lane_off_v)
                                   : lookup_column<3>(lut_v, src, lane_off_v);
            }
        };
        __builtin_amdgcn_sched_barrier(0);
        float4v acc[2];
        float4v acc_s[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            acc[b] = float4v{0.f, 0.f, 0.f, 0.f};
            acc_s[b] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ka[b][ks]), qh[ks], acc[b], 0, 0, 0);
            if constexpr (PROD) {
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    const uint4v sg = sign_operand(kw[b][ks], 0x3C003C00u);
                    acc_s[b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, sg), qsh[ks], acc_s[b], 0, 0, 0);
                }
            }
            if (b == 0) v_group(0, vb[0]);
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (D256) {
            // ---- the other half of the head's coordinates: wavefront h ^ 1 has their part of every score.  Each
            // posts its part (times its own query scale) in its patch of LDS behind the tile slots and adds the
            // partner's: a + b in one wavefront, b + a in the other, the same bits.  The patch is rewritten
            // every tile, so a wavefront waits for the partner to have read the tile before (bounded waits).
            float4v* xb = reinterpret_cast<float4v*>(slots + 2 * kTileBytes);
            const int hp = h ^ 1;
            if (!lds_flag_wait(&xflags[8 + hp], uint32_t(it), p.spin_limit)) { flags[2] = 1u; handoff_failed = true; }
            const float4v m0 = acc[0] * qscale, m1 = acc[1] * qscale;
            xb[(2 * h) * kWave + lane] = m0;
            xb[(2 * h + 1) * kWave + lane] = m1;
            lds_flag_signal(&xflags[h], lane);
            if (!lds_flag_wait(&xflags[hp], uint32_t(it) + 1u, p.spin_limit)) { flags[2] = 1u; handoff_failed = true; }
            const float4v o0 = xb[(2 * hp) * kWave + lane], o1 = xb[(2 * hp + 1) * kWave + lane];
            acc[0] = m0 + o0;
            acc[1] = m1 + o1;
            lds_flag_signal(&xflags[8 + h], lane);
        }

        // ---- this lane's scores ------------------------------------------------------------------
        float a_[NSC], rv[NSC];
#pragma unroll
        for (int e = 0; e < NSC; ++e) {
            float s, s2 = 0.0f;
            if (GP == 4) {
                const float s0 = (cls & 1) ? acc[0][2 + e] : acc[0][e];
                const float s1 = (cls & 1) ? acc[1][2 + e] : acc[1][e];
                s = (cls >> 1) ? s1 : s0;
                if (PROD) {
                    const float u0 = (cls & 1) ? acc_s[0][2 + e] : acc_s[0][e];
                    const float u1 = (cls & 1) ? acc_s[1][2 + e] : acc_s[1][e];
                    s2 = (cls >> 1) ? u1 : u0;
                }
            } else if (GP == 8) {
                s = cls ? acc[1][e] : acc[0][e];
                if (PROD) s2 = cls ? acc_s[1][e] : acc_s[0][e];
            } else {
                s = acc[e >> 2][e & 3];
                if (PROD) s2 = acc_s[e >> 2][e & 3];
            }
            const bool live = t0 + sc_tok[e] < end_mine;
            rv[e] = live ? vn[e] : 0.0f;
            float sc = D256 ? s * kn[e] : s * kn[e] * qscale;      // D256: the scale went in before the halves were added
            if (PROD) sc = __builtin_fmaf(s2 * kg[e], qscale_s, sc);
            a_[e] = live ? sc : -__builtin_inff();
        }
        // Weights relative to the reference M the head already has.  M is not the exact running
        // maximum: it moves only when a score leads it by more than 2^16 or a weighted value norm
        // w * |v| would not fit fp16 (the P operand), which one vote over the wavefront finds out.
        // Any reference gives the same softmax as long as numerator and denominator share it.
        float wv[NSC];
        float psum = 0.0f;
        bool redo = false;
#pragma unroll
        for (int e = 0; e < NSC; ++e) {
            const float d = a_[e] - M;
            const float w = __builtin_amdgcn_exp2f(d);
            psum += w;
            wv[e] = w * rv[e];
            // (MULTI > 0: the first tile of a split may hold no token of this wavefront; -inf - -inf
            // is then NaN in every lane, and the vote must still send the tile through the safe path)
            redo = redo || (MULTI > 0 ? !(d <= kMaxLead) : d > kMaxLead) || wv[e] > kHalfSafe;
        }
        if (__any(redo)) {
            // The reference moves to max(M, max over the tile of (score + bias)), where the bias of a
            // token is the number of binary orders its value norm lies above 2^10: weights then stay
            // below 1 / 2^bias and w * |v| below 2^11 whatever the norms are.
            float tmax = -__builtin_inff();
#pragma unroll
            for (int e = 0; e < NSC; ++e) tmax = __builtin_fmaxf(tmax, a_[e] + norm_bias(rv[e]));
            tmax = max_same_head<GP>(tmax);
            const float Mnew = __builtin_fmaxf(M, tmax);
            const float Ms = Mnew == -__builtin_inff() ? 0.0f : Mnew;
            const float alpha = __builtin_amdgcn_exp2f(M - Ms);   // M = -inf (first tile): 0
            M = Mnew;
            psum = 0.0f;
#pragma unroll
            for (int e = 0; e < NSC; ++e) {
                const float w = __builtin_amdgcn_exp2f(a_[e] - Ms);
                psum += w;
                wv[e] = __builtin_fminf(w * rv[e], kHalfMax);     // only a norm of Inf still reaches the bound
            }
            lsum *= alpha;
            float ar[4];
            if (GP == 4) {
                ar[0] = dpp_mov<0x00>(alpha);
                ar[1] = dpp_mov<0x55>(alpha);
                ar[2] = dpp_mov<0xAA>(alpha);
                ar[3] = dpp_mov<0xFF>(alpha);
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) ar[i] = __shfl(alpha, 4 * g + i, kWave);
            }
#pragma unroll
            for (int db = 0; db < DPL; ++db)
#pragma unroll
                for (int i = 0; i < 4; ++i) O[db][i] *= ar[i];
        }
        lsum += psum;

        // ---- weights as the A operand: slot j <-> (block j / 4, row 4g + j % 4) -------------------
        // (the weights of this lane are packed once and placed with lane-constant masks)
        uint32_t pk[NSC / 2];
#pragma unroll
        for (int e = 0; e < NSC / 2; ++e) {
            const half2v h2 = {_Float16(wv[2 * e]), _Float16(wv[2 * e + 1])};
            pk[e] = __builtin_bit_cast(uint32_t, h2);
        }
        uint4v pa_w;
        if (GP == 16) {
            pa_w = uint4v{pk[0], pk[1 % (NSC / 2)], pk[2 % (NSC / 2)], pk[3 % (NSC / 2)]};
        } else {
            pa_w = uint4v{pk[0] & pa_mask[0], pk[1 % (NSC / 2)] & pa_mask[1], pk[0] & pa_mask[2], pk[1 % (NSC / 2)] & pa_mask[3]};
        }
        const half8 pa = __builtin_bit_cast(half8, pa_w);

        // ---- O += P . V ------------------------------------------------------------------------------
        __builtin_amdgcn_sched_barrier(0);
        v_group(1, vb[1]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            O[e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, __builtin_bit_cast(half8, vb[0][e]), O[e], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            O[4 + e] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, __builtin_bit_cast(half8, vb[1][e]), O[4 + e], 0, 0, 0);
    };

    // ---- tiles ------------------------------------------------------------------------------------
    if constexpr (CW == 0) {
        write_slot(0);                            // tile 0, loaded before the query was prepared
        issue_loads(clamp_t0(begin + 32));
        int i = 0;
        for (int t0 = begin; t0 < end; t0 += 32, ++i) {
            __syncthreads();                      // tile i is in LDS; slot of tile i - 1 is free
            write_slot((i + 1) & 1);              // tile i + 1 (its loads ran during tile i - 1)
            issue_loads(clamp_t0(t0 + 64));       // tile i + 2
            compute_tile(t0, i & 1, i);
        }
    } else {
        int i = 0;
        for (int t0 = begin; t0 < end; t0 += 32, ++i) {
            // consumer side: tile i is complete when every copy wavefront has written its part of it
            if (!lds_flag_wait(&flags[3 + (i & 1)], uint32_t(CW) * uint32_t((i >> 1) + 1), p.spin_limit)) {
                flags[2] = 1u;
                handoff_failed = true;
            }
            compute_tile(t0, i & 1, i);
            if constexpr (STORE) {
                if (i == 0 && stores_token && last_t0 >= begin + 64) {      // (see the prologue)
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
                    lds_flag_signal(&flags[7], lane);
                }
            }
        }
    }

    // ---- publish the partial of this split (as in the direct kernel) -----------------------------
    auto sum_xor = [](float v, int mask) {
        return mask == 16 ? sum_xor16(v) : (mask == 32 ? sum_xor32(v) : v + xor_shuffle(v, mask));
    };
#pragma unroll
    for (int mask = GP; mask < 64; mask <<= 1) lsum = sum_xor(lsum, mask);
#pragma unroll
    for (int db = 0; db < DPL; ++db)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = O[db][i];
#pragma unroll
            for (int mask = 4 * GP; mask < 64; mask <<= 1) v = sum_xor(v, mask);
            O[db][i] = v;
        }
    if constexpr (LINEAR) {
        // the partials of the wavefronts go through the tile slots: every computing wavefront must have fetched its
        // operands of the last tiles (tile i lies in slot i % 2)
        const int ntiles = (end - begin + 31) >> 5;
        if (!lds_flag_wait(&flags[5], 8u * uint32_t((ntiles + 1) >> 1), p.spin_limit) ||
            !lds_flag_wait(&flags[6], 8u * uint32_t(ntiles >> 1), p.spin_limit)) {
            flags[2] = 1u;
            handoff_failed = true;
        }
    }
    if constexpr (CW > 0) {
        // a hand-off that timed out, in the prologue or in the tile loop: the result cannot be
        // trusted, so it is made NaN and the fault is counted
        if (handoff_failed ||
            __builtin_amdgcn_readfirstlane(__hip_atomic_load(&flags[2], __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_WORKGROUP)) != 0u) {
            M = __builtin_nanf("");
            if (handoff_failed && lane == 0) atomicAdd(&g_decode_faults, 1u);
        }
    }
    if constexpr (LINEAR) {
        // The TPR wavefronts of a head hold the partials of its tokens t mod TPR of every row.  They are merged here
        // into the one partial of the split: each posts its own in LDS, and each then combines its share of the
        // coordinates (128 / TPR of every query head) from all of them.
        float* xacc = reinterpret_cast<float*>(slots);        // [wavefront][query head 0..15][128]
        float* xml = xacc + 8 * 16 * 128;                     // [wavefront][query head][maximum, denominator]
        if (g == 0 && n < p.G) {
            xml[(h * 16 + n) * 2] = M;
            xml[(h * 16 + n) * 2 + 1] = lsum;
        }
        if (g < GP / 4) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int head = 4 * g + i;
                if (head < p.G) {
                    float* dst = xacc + (h * 16 + head) * 128 + n * DPL;
#pragma unroll
                    for (int q4 = 0; q4 < DPL / 4; ++q4)
                        *reinterpret_cast<float4v*>(dst + 4 * q4) = float4v{O[4 * q4][i], O[4 * q4 + 1][i], O[4 * q4 + 2][i], O[4 * q4 + 3][i]};
                }
            }
        }
        lds_flag_signal(&xflags[16], lane);
        bool merged = lds_flag_wait(&xflags[16], 8u, p.spin_limit);
        if (!merged && lane == 0) atomicAdd(&g_decode_faults, 1u);
        constexpr int CPW = 128 / TPR;                        // coordinates of a head that this wavefront combines
        // maximum over the wavefronts of this head (NaN when a hand-off failed), no array: the values are read again
        auto merged_max = [&](int head) __attribute__((always_inline)) -> float {
            float ms = -__builtin_inff();
            bool bad = !merged;
#pragma unroll
            for (int t = 0; t < TPR; ++t) {
                const float m = xml[((t * HPR + hh) * 16 + head) * 2];
                bad = bad || m != m;
                ms = __builtin_fmaxf(ms, m);
            }
            return bad ? __builtin_nanf("") : ms;
        };
        for (int idx = lane; idx < p.G * CPW; idx += kWave) {
            const int head = idx / CPW, c = CPW * tsel + (idx - head * CPW);
            const float ms = merged_max(head);
            float acc = 0.0f;
#pragma unroll
            for (int t = 0; t < TPR; ++t) {
                const float m = xml[((t * HPR + hh) * 16 + head) * 2];
                const float w = ms == -__builtin_inff() ? 0.0f : __builtin_amdgcn_exp2f(m - ms);
                acc += w * xacc[((t * HPR + hh) * 16 + head) * 128 + c];
            }
            if constexpr (D64) {     // a query head's output: the half of the 128 coordinates that is its own head's
                if ((c >> 6) == (head >= p.G / 2 ? 1 : 0))
                    p.part_acc[((int64_t(seq) * p.H_Q + hq0 + hr * p.G + head) * NS + split) * 64 + (c & 63)] = acc;
            } else if constexpr (D256) {   // this wavefront's half of the head's 256 coordinates
                p.part_acc[((int64_t(seq) * p.H_Q + hq0 + hr * p.G + head) * NS + split) * 256 + 128 * (h & 1) + c] = acc;
            } else {
                p.part_acc[((int64_t(seq) * p.H_Q + hq0 + hr * p.G + head) * NS + split) * D + c] = acc;
            }
        }
        if (tsel == 0 && lane < p.G && (!D256 || (h & 1) == 0)) {
            const float ms = merged_max(lane);
            float l = 0.0f;
#pragma unroll
            for (int t = 0; t < TPR; ++t) {
                const float m = xml[((t * HPR + hh) * 16 + lane) * 2];
                const float w = ms == -__builtin_inff() ? 0.0f : __builtin_amdgcn_exp2f(m - ms);
                l += w * xml[((t * HPR + hh) * 16 + lane) * 2 + 1];
            }
            const int64_t o = (int64_t(seq) * p.H_Q + hq0 + hr * p.G + lane) * NS + split;
            p.part_m[o] = ms;
            p.part_l[o] = l;
        }
        return;
    }
    if (g == 0 && n < p.G && (!D256 || (h & 1) == 0)) {        // D256: both halves hold the same maximum and denominator
        const int64_t o = (int64_t(seq) * p.H_Q + hq0 + hq_lane) * NS_out + split_out;
        p.part_m[o] = M;
        p.part_l[o] = lsum;
    }
    if (g < GP / 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int head = 4 * g + i;
            // D64: a query head's output is the half of the 128 coordinates that belongs to its own head of 64
            const bool mine = !D64 || (n >> 3) == (head >= p.G / 2 ? 1 : 0);
            if (head < p.G && mine) {
                float* dst = D64 ? p.part_acc + ((int64_t(seq) * p.H_Q + hq0 + hr * p.G + head) * NS_out + split_out) * 64 + (n & 7) * DPL
                           : D256 ? p.part_acc + ((int64_t(seq) * p.H_Q + hq0 + hr * p.G + head) * NS_out + split_out) * 256 + 128 * (h & 1) + n * DPL
                                  : p.part_acc + ((int64_t(seq) * p.H_Q + hq0 + hr * p.G + head) * NS_out + split_out) * D + n * DPL;
#pragma unroll
                for (int q4 = 0; q4 < DPL / 4; ++q4) {
                    const float4v v = {O[4 * q4][i], O[4 * q4 + 1][i], O[4 * q4 + 2][i], O[4 * q4 + 3][i]};
                    *reinterpret_cast<float4v*>(dst + 4 * q4) = v;
                }
            }
        }
    }
}

// q_rot[row, j] = sum_k q[row, k] * R[j, k], rounded to the query dtype
// (src/flashquant/kernels/paged_decode.py:113).  rows = num_seqs * H_Q.
template <int D, int DT>
__global__ __launch_bounds__(256) void rotate_q_kernel(const uint16_t* __restrict__ q, const float* __restrict__ R,
                                                       uint16_t* __restrict__ q_rot, int64_t rows, int col_major) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int64_t row0 = int64_t(blockIdx.x) * kRotRows;
    const int64_t my_row = row0 + n < rows ? row0 + n : rows - 1;
    float a[D / 32][8];
#pragma unroll
    for (int j = 0; j < D / 32; ++j) {
        const uint4v raw = *reinterpret_cast<const uint4v*>(q + my_row * D + 32 * j + 8 * g);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[j][2 * i] = load_elem<DT>(uint16_t(w[i] & 0xffffu));
            a[j][2 * i + 1] = load_elem<DT>(uint16_t(w[i] >> 16));
        }
    }
    // gridDim.y workgroups share the column blocks of a row group (one round of four blocks each at head_dim 256:
    // the rows are few, 1024 in a decode step of 32 sequences x 32 heads, and the matrix is what is fetched)
    for (int cb = wave + 4 * int(blockIdx.y); cb < D / 16; cb += 4 * int(gridDim.y)) {
        float b[D / 32][8];
        load_rotation_any<D>(R, col_major != 0, true, 16 * cb, n, g, b);
        const float4v acc = rotate_block<D>(a, b);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int64_t row = row0 + 4 * g + i;
            if (row < rows) q_rot[row * D + 16 * cb + n] = store_elem<DT>(acc[i]);
        }
    }
}

// Combine of the split partials: out_rot = sum_s acc_s 2^(m_s - m*) / sum_s l_s 2^(m_s - m*)
// (0 when every split is empty), rounded to the query dtype as the reference's
// rotated-space result is (cpu_reference.py:366), then multiplied by R in float32 and
// rounded again (paged_decode.py:123).  rows = num_seqs * H_Q; a workgroup owns RW rows
// (4, 8 or 16: the fewer, the more workgroups share the combine, the more often the matrix is
// fetched): 256 / RW threads combine a row into LDS, then all rotate from there.
// CS: the output columns of a row group are shared by CS workgroups (blockIdx.y), each combining the rows for
// itself and fetching 1 / CS of the matrix: at head_dim 256 the matrix is 256 KB, and a workgroup that fetches all
// of it holds 256 matrix values per lane.
template <int D, int DT, int RW, int CS = 1>
__global__ __launch_bounds__(256) void reduce_rotate_kernel(const float* __restrict__ part_acc,
                                                            const float* __restrict__ part_m,
                                                            const float* __restrict__ part_l,
                                                            const float* __restrict__ R, uint16_t* __restrict__ out,
                                                            int64_t rows, int NS, int col_major) {
    static_assert((D / 64) % CS == 0, "whole rounds of column blocks per workgroup");
    constexpr int CBW = D / 64 / CS;       // 16-column blocks per wavefront
    const int cb0 = 4 * CBW * int(blockIdx.y);     // first column block of this workgroup
    constexpr int OSTRIDE = D + 8;         // 16-bit words per staged row (padded: conflict-free operand reads)
    constexpr int TPR = 256 / RW;          // threads that combine one row
    constexpr int CPT = D / TPR < 2 ? 2 : D / TPR;      // coordinates per thread and pass (2, 4 or 8)
    constexpr int ACTIVE = D / CPT < TPR ? D / CPT : TPR;   // threads of a row that have coordinates
    static_assert(CPT <= 8, "a thread stages at most eight coordinates of a row (head_dim 256: at most 8 rows a workgroup)");
    __shared__ __attribute__((aligned(16))) uint16_t os[RW * OSTRIDE];   // combined rows, query dtype
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    const int64_t row0 = int64_t(blockIdx.x) * RW;

    // ---- combine: the loads of up to eight splits (maximum, denominator, accumulator) are all in
    // flight together; they are asked for before the matrix, which is needed later ------------------
    const int r = threadIdx.x / TPR, t = threadIdx.x % TPR;
    const int64_t row = row0 + r < rows ? row0 + r : rows - 1;
    const int64_t base = row * NS;
    float mstar = -__builtin_inff();
    bool poisoned = false;      // a split published NaN as its maximum: its workgroup could not vouch for it
    // bit c: the chunk of eight splits c (mod 64) holds a split that wrote something.  Splits
    // beyond a sequence's length are empty (m = -inf), whole chunks of them when the split count
    // was chosen for the longest possible context: those are not read at all.
    uint64_t live_chunks = ~0ull;
    if (NS > 8) {
        // the threads of a row share the maxima: thread t reads those of splits t, t + TPR, ...,
        // four at a time, so that 4 TPR splits cost one round trip
        uint32_t live_lo = 0u, live_hi = 0u;
        for (int s0 = 0; s0 < NS; s0 += 4 * TPR) {
            float mv[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int idx = s0 + t + TPR * k;
                mv[k] = part_m[base + (idx < NS ? idx : NS - 1)];
            }
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int idx = s0 + t + TPR * k;
                const bool wrote = idx < NS && mv[k] != -__builtin_inff();
                poisoned = poisoned || (idx < NS && mv[k] != mv[k]);
                mstar = wrote ? __builtin_fmaxf(mstar, mv[k]) : mstar;
                const int chunk = (idx >> 3) & 63;
                live_lo |= (wrote && chunk < 32) ? 1u << chunk : 0u;
                live_hi |= (wrote && chunk >= 32) ? 1u << (chunk - 32) : 0u;
            }
        }
#pragma unroll
        for (int mask = 1; mask < TPR; mask <<= 1) {
            mstar = __builtin_fmaxf(mstar, xor_shuffle(mstar, mask));
            poisoned = poisoned || __shfl_xor(int(poisoned), mask, kWave) != 0;
            live_lo |= uint32_t(__shfl_xor(int(live_lo), mask, kWave));
            live_hi |= uint32_t(__shfl_xor(int(live_hi), mask, kWave));
        }
        live_chunks = (uint64_t(live_hi) << 32) | live_lo;
    }
    float num[CPT];
#pragma unroll
    for (int e = 0; e < CPT; ++e) num[e] = 0.0f;
    float den = 0.0f;
    const int c0 = CPT * (t < ACTIVE ? t : 0);
    for (int s0 = 0; s0 < NS; s0 += 8) {
        if (!((live_chunks >> ((s0 >> 3) & 63)) & 1ull)) continue;
        float mv[8], lv[8];
        float pv[8][CPT];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int sidx = s0 + k < NS ? s0 + k : NS - 1;
            mv[k] = part_m[base + sidx];
            lv[k] = part_l[base + sidx];
            // An empty split (m = -inf) never wrote its accumulator; it is read all the same
            // (and ignored below), so that no load has to wait for another one.
            const float* src = part_acc + (base + sidx) * D + c0;
            if constexpr (CPT == 2) {
                const float2v v = *reinterpret_cast<const float2v*>(src);
                pv[k][0] = v.x; pv[k][1] = v.y;
            } else {
#pragma unroll
                for (int q4 = 0; q4 < CPT / 4; ++q4) {
                    const float4v v = reinterpret_cast<const float4v*>(src)[q4];
                    pv[k][4 * q4] = v.x; pv[k][4 * q4 + 1] = v.y; pv[k][4 * q4 + 2] = v.z; pv[k][4 * q4 + 3] = v.w;
                }
            }
        }
        if (NS <= 8) {
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                mstar = __builtin_fmaxf(mstar, mv[k]);
                poisoned = poisoned || mv[k] != mv[k];
            }
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const bool use = s0 + k < NS && mv[k] != -__builtin_inff();
            const float w = use ? __builtin_amdgcn_exp2f(mv[k] - mstar) : 0.0f;
            den = __builtin_fmaf(lv[k], w, den);
            // a weight of 0 must also silence a NaN or Inf in memory that no split wrote
#pragma unroll
            for (int e = 0; e < CPT; ++e) num[e] = use ? __builtin_fmaf(pv[k][e], w, num[e]) : num[e];
        }
    }
    // the matrix columns of this wavefront: asked for behind the partials, they arrive during the combine
    float rbv[CBW][D / 32][8];
    if (R != nullptr) {
#pragma unroll
        for (int i = 0; i < CBW; ++i) load_rotation_any<D>(R, col_major != 0, false, 16 * (cb0 + wave + 4 * i), n, g, rbv[i]);
    }
    {
        const bool live = row0 + r < rows && den > 0.0f;
        const float inv = live ? 1.0f / den : 0.0f;
        uint32_t wds[CPT / 2];
#pragma unroll
        for (int e = 0; e < CPT / 2; ++e) {
            // a poisoned row comes out NaN, never as a plausible number
            const uint32_t a0 = poisoned ? store_elem<DT>(__builtin_nanf("")) : (live ? store_elem<DT>(num[2 * e] / den) : 0u);
            const uint32_t a1 = poisoned ? store_elem<DT>(__builtin_nanf("")) : (live ? store_elem<DT>(num[2 * e + 1] / den) : 0u);
            wds[e] = a0 | (a1 << 16);
        }
        (void)inv;
        if (t < ACTIVE) {
            if constexpr (CPT == 2) *reinterpret_cast<uint32_t*>(&os[r * OSTRIDE + c0]) = wds[0];
            else if constexpr (CPT == 4) *reinterpret_cast<uint2v*>(&os[r * OSTRIDE + c0]) = uint2v{wds[0], wds[1]};
            else *reinterpret_cast<uint4v*>(&os[r * OSTRIDE + c0]) = uint4v{wds[0], wds[1], wds[2], wds[3]};
        }
    }
    __syncthreads();
    if (R == nullptr) {
        if (CS > 1 && blockIdx.y != 0) return;        // no rotation: one workgroup writes the combined rows
        for (int c = threadIdx.x; c < RW * (D / 8); c += 256) {
            const int rr = c / (D / 8), q = c % (D / 8);
            const int64_t orow = row0 + rr;
            if (orow < rows) reinterpret_cast<uint4v*>(out + orow * D)[q] = *reinterpret_cast<const uint4v*>(&os[rr * OSTRIDE + 8 * q]);
        }
        return;
    }
    // ---- rotate back on the fp16 MFMA: the rows are exact in fp16 up to a power of two.  With fewer
    // than 16 rows the operand rows repeat (row n % RW) and only the first RW result rows are kept. ----
    uint4v raw[D / 32];
#pragma unroll
    for (int j = 0; j < D / 32; ++j) raw[j] = *reinterpret_cast<const uint4v*>(&os[(n % RW) * OSTRIDE + 32 * j + 8 * g]);
    half8 a[D / 32];
    float up;
    rows_as_f16<D, DT>(raw, a, up);
#pragma unroll
    for (int i = 0; i < CBW; ++i) {
        half8 rhi[D / 32], rlo[D / 32];
        split_rotation_block<D>(rbv[i], rhi, rlo);
        const float4v acc = rotate_block_f16<D>(a, rhi, rlo);
        const int cb = cb0 + wave + 4 * i;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int rr = 4 * g + k;
            const int64_t orow = row0 + rr;
            if (rr < RW && orow < rows) out[orow * D + 16 * cb + n] = store_elem<DT>(acc[k] * up);
        }
    }
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

struct WorkspaceLayout {
    size_t acc, m, l, qrot, total;
};
inline WorkspaceLayout workspace_layout(int S, int H_Q, int D, int NS) {
    WorkspaceLayout w;
    const size_t rows = size_t(S) * H_Q;
    w.acc = 0;
    w.m = align_up(w.acc + rows * NS * D * sizeof(float), 256);
    w.l = align_up(w.m + rows * NS * sizeof(float), 256);
    w.qrot = align_up(w.l + rows * NS * sizeof(float), 256);
    w.total = align_up(w.qrot + rows * D * 2, 256);
    return w;
}


// Workgroups that run at a time (one per CU) when the staged kernel should size its chunks from
// the actual sequence lengths, 0 when the fixed chunks already fill the chip in one round or the
// batch is too large for one lane per sequence.
inline int staged_balance_slots(int num_seqs, int num_splits) {
    const int cus = fq_host::device_cu_count();
    return (num_seqs <= 64 && int64_t(num_seqs) * num_splits > cus) ? cus : 0;
}

// The kernel-variant switches as one decode call sees them.  They are process-wide and may be changed
// by another thread at any time (fq_set_option): a call reads them once, here, and everything that
// depends on them (which kernel runs, how many partials it writes, how the workspace is laid out, how
// many the combine kernel merges) is derived from this one reading.
struct DecodeVariant {
    bool direct;        // FQ_OPT_DECODE_DIRECT
    bool ring;          // FQ_OPT_DECODE_RING
    int copy_waves;     // 4 or 0 (FQ_OPT_DECODE_COPY_WAVES)
};
inline DecodeVariant read_decode_variant() {
    DecodeVariant v;
    v.direct = fq_host::option(FQ_OPT_DECODE_DIRECT) != 0;
    v.ring = fq_host::option(FQ_OPT_DECODE_RING) != 0;
    v.copy_waves = fq_host::option(FQ_OPT_DECODE_COPY_WAVES) != 0 ? 4 : 0;
    return v;
}

// The new token of a serving step, for the staged kernel that stores it (DecodeParams: new_key ...).
struct NewToken {
    const void* key;
    const void* value;
    const int64_t* slots;
    const float* boundaries;
    uint8_t* cache;
};

// The staged kernel covers KV heads of dimension 128 in groups of 8.
inline bool staged_applies(int D, int H_KV, const DecodeVariant& v) {
    return D == 128 && H_KV >= 8 && H_KV % 8 == 0 && !v.direct;
}

template <bool PROD, typename K>
int launch_staged(K kernel, const DecodeParams& p, int S, hipStream_t stream, int copy_waves = 0) {
    // dynamic part only; the 64 KB table is static
    const size_t lds = 2 * size_t(StagedCfg<PROD>::TILE_BYTES);
    return launch_with_lds(kernel, p, dim3(S, p.num_splits, p.H_KV / 8), dim3(512 + 64 * copy_waves), lds, stream);
}

// The staged kernel runs with four more wavefronts that only copy; the switch
// FQ_OPT_DECODE_COPY_WAVES = 0 selects the form in which the eight wavefronts copy and compute in turn.

// Staged kernel for every page size and group size; PROD selects the TurboQuantProd page format.
template <int DT, bool PROD>
int launch_staged_any(const DecodeParams& p, int S, int BS, bool wide, hipStream_t stream, int copy_waves,
                      bool store = false) {
#define FQ_STAGED_GP(BSL, GPV)                                                                                  \
    /* TurboQuantProd pages come with at most 64 query heads (8 per KV head) */                                 \
    if constexpr (PROD && GPV == 16) return FQ_ERR_BAD_SHAPE;                                                   \
    else {                                                                                                      \
        if constexpr (!PROD) {                                                                                  \
            if (store) {                                                                                        \
                if (copy_waves != 4) return FQ_ERR_LAUNCH;                                                      \
                return launch_staged<PROD>(paged_decode_staged_kernel<BSL, GPV, DT, 4, PROD, 4, false, true>, p, S, stream, 4); \
            }                                                                                                   \
        }                                                                                                       \
        if (copy_waves == 4)                                                                                    \
            return (wide || PROD) ? launch_staged<PROD>(paged_decode_staged_kernel<BSL, GPV, DT, 4, PROD, 4>, p, S, stream, 4) \
                                  : launch_staged<PROD>(paged_decode_staged_kernel<BSL, GPV, DT, PROD ? 4 : 1, PROD, 4>, p, S, stream, 4); \
        return launch_staged<PROD>(paged_decode_staged_kernel<BSL, GPV, DT, 4, PROD, 0>, p, S, stream); \
    }
#define FQ_STAGED_BS(BSL)                         \
    do {                                          \
        if (p.G <= 4) { FQ_STAGED_GP(BSL, 4); }   \
        else if (p.G <= 8) { FQ_STAGED_GP(BSL, 8); } \
        else { FQ_STAGED_GP(BSL, 16); }           \
    } while (0)
    switch (BS) {
        case 8: FQ_STAGED_BS(3); break;
        case 16: FQ_STAGED_BS(4); break;
        default: FQ_STAGED_BS(5); break;
    }
#undef FQ_STAGED_BS
#undef FQ_STAGED_GP
    return FQ_ERR_UNSUPPORTED_BLOCK;
}

// 1, 2 or 4 KV heads of dimension 128 on pages of 16 or 32 tokens: the staged kernel on rows of 8, 4 or 2 tokens kept
// in LDS as they lie in the cache (`rows_per_page` = block_size * H_KV / 8); the wavefronts that share a head (one per
// token of a row) merge their partials before they leave the workgroup.
inline bool staged_linear_applies(int D, int H_KV, int block_size, const DecodeVariant& v) {
    return D == 128 && (H_KV == 1 || H_KV == 2 || H_KV == 4) && block_size >= 16 && !v.direct && v.copy_waves == 4;
}
template <int DT>
int launch_staged_linear(const DecodeParams& p, int S, int rows_per_page, hipStream_t stream) {
    const size_t lds = 2 * 32 * 1104;         // two tiles of 32 rows, a row every 1104 bytes
    const dim3 grid(S, p.num_splits, 1), block(512 + 64 * 4);
    const bool store = p.new_key != nullptr;
#define FQ_LINEAR_GP(BSL, GPV, MULTIV)                                                                                \
    if (store)                                                                                                        \
        return launch_with_lds(paged_decode_staged_kernel<BSL, GPV, DT, 4, false, 4, MULTIV, true>, p, grid, block, lds, stream); \
    return launch_with_lds(paged_decode_staged_kernel<BSL, GPV, DT, 4, false, 4, MULTIV>, p, grid, block, lds, stream)
#define FQ_LINEAR_BS(BSL, MULTIV)                            \
    do {                                                     \
        if (p.G <= 4) { FQ_LINEAR_GP(BSL, 4, MULTIV); }      \
        else if (p.G <= 8) { FQ_LINEAR_GP(BSL, 8, MULTIV); } \
        else { FQ_LINEAR_GP(BSL, 16, MULTIV); }              \
    } while (0)
    if (p.H_KV == 1) {
        if (rows_per_page == 2) FQ_LINEAR_BS(1, 3);
        else FQ_LINEAR_BS(2, 3);
    } else if (p.H_KV == 2) {
        if (rows_per_page == 4) FQ_LINEAR_BS(2, 2);
        else FQ_LINEAR_BS(3, 2);
    } else {
        if (rows_per_page == 8) FQ_LINEAR_BS(3, 4);
        else FQ_LINEAR_BS(4, 4);
    }
#undef FQ_LINEAR_BS
#undef FQ_LINEAR_GP
}

// head_dim 64 on the staged kernel: pairs of neighbouring KV heads as heads of 128 (16 real heads a group), or, with
// 8, 4 or 2 KV heads on pages of 16 or 32 tokens, rows of 2, 4 or 8 tokens of 4, 2 or 1 such pairs.  Up to 8 query
// heads per KV head.
inline bool staged_d64_full_applies(int D, int H_KV, int G, const DecodeVariant& v) {
    return D == 64 && H_KV % 16 == 0 && G <= 8 && !v.direct && v.copy_waves == 4;
}
inline bool staged_d64_half_applies(int D, int H_KV, int G, int block_size, const DecodeVariant& v) {
    return D == 64 && (H_KV == 8 || H_KV == 4 || H_KV == 2) && G <= 8 && block_size >= 16 && !v.direct && v.copy_waves == 4;
}
template <int DT>
int launch_staged_d64(const DecodeParams& p, int S, int rows_per_page, bool wide, bool half, hipStream_t stream) {
    // (rows of two tokens: as they lie in the cache, a row every 1168 bytes)
    const size_t lds = half ? 2 * 32 * 1168 : 2 * size_t(StagedCfg<false, 64>::TILE_BYTES);
    const dim3 grid(S, p.num_splits, half ? 1 : p.H_KV / 16), block(512 + 64 * 4);
#define FQ_D64_GP(BSL, GPV, MULTIV)                                                                                \
    return launch_with_lds(paged_decode_staged_kernel<BSL, GPV, DT, 4, false, 4, MULTIV, false, 64>, p, grid, block, lds, stream)
#define FQ_D64_BS(BSL, MULTIV)                            \
    do {                                                 \
        if (p.G <= 4) { FQ_D64_GP(BSL, 4, MULTIV); }      \
        else if (p.G <= 8) { FQ_D64_GP(BSL, 8, MULTIV); } \
        else { FQ_D64_GP(BSL, 16, MULTIV); }              \
    } while (0)
    const bool store = p.new_key != nullptr;     // (rows of tokens only)
    if (half && p.H_KV == 8 && !store) {
        if (rows_per_page == 8) FQ_D64_BS(3, 4);
        else FQ_D64_BS(4, 4);
    } else if (half && store) {
#define FQ_D64_STORE(BSL, MULTIV)                                                                                                        \
    do {                                                                                                                                 \
        if (p.G <= 4) return launch_with_lds(paged_decode_staged_kernel<BSL, 4, DT, 4, false, 4, MULTIV, true, 64>, p, grid, block, lds, stream);   \
        if (p.G <= 8) return launch_with_lds(paged_decode_staged_kernel<BSL, 8, DT, 4, false, 4, MULTIV, true, 64>, p, grid, block, lds, stream);   \
        return launch_with_lds(paged_decode_staged_kernel<BSL, 16, DT, 4, false, 4, MULTIV, true, 64>, p, grid, block, lds, stream);     \
    } while (0)
        if (p.H_KV == 8) {
            if (rows_per_page == 8) FQ_D64_STORE(3, 4);
            else FQ_D64_STORE(4, 4);
        } else if (p.H_KV == 4) {
            if (rows_per_page == 4) FQ_D64_STORE(2, 2);
            else FQ_D64_STORE(3, 2);
        } else {
            if (rows_per_page == 2) FQ_D64_STORE(1, 3);
            else FQ_D64_STORE(2, 3);
        }
#undef FQ_D64_STORE
    } else if (half) {      // 4 and 2 KV heads: always four page-id registers
#define FQ_D64_FEW(BSL, MULTIV)                                                                                                          \
    do {                                                                                                                                 \
        if (p.G <= 4) return launch_with_lds(paged_decode_staged_kernel<BSL, 4, DT, 4, false, 4, MULTIV, false, 64>, p, grid, block, lds, stream);  \
        if (p.G <= 8) return launch_with_lds(paged_decode_staged_kernel<BSL, 8, DT, 4, false, 4, MULTIV, false, 64>, p, grid, block, lds, stream);  \
        return launch_with_lds(paged_decode_staged_kernel<BSL, 16, DT, 4, false, 4, MULTIV, false, 64>, p, grid, block, lds, stream);    \
    } while (0)
        if (p.H_KV == 4) {
            if (rows_per_page == 4) FQ_D64_FEW(2, 2);
            else FQ_D64_FEW(3, 2);
        } else {
            if (rows_per_page == 2) FQ_D64_FEW(1, 3);
            else FQ_D64_FEW(2, 3);
        }
#undef FQ_D64_FEW
    } else {
        if (rows_per_page == 8) FQ_D64_BS(3, 0);
        else if (rows_per_page == 16) FQ_D64_BS(4, 0);
        else FQ_D64_BS(5, 0);
    }
#undef FQ_D64_BS
#undef FQ_D64_GP
}

// head_dim 256 on the staged kernel: every KV head as two heads of 128, 4 real heads a group; the query comes rotated.
inline bool staged_d256_applies(int D, int H_KV, const DecodeVariant& v) {
    return D == 256 && H_KV % 4 == 0 && !v.direct && v.copy_waves == 4;
}
template <int DT>
int launch_staged_d256(const DecodeParams& p, int S, int BS, bool wide, hipStream_t stream) {
    // two tile slots and the patch through which the halves of a head exchange their scores
    const size_t lds = 2 * size_t(StagedCfg<false, 256>::TILE_BYTES) + 8 * 2 * kWave * sizeof(float4v);
    const dim3 grid(S, p.num_splits, p.H_KV / 4), block(512 + 64 * 4);
#define FQ_D256_GP(BSL, GPV)                                                                                       \
    return launch_with_lds(paged_decode_staged_kernel<BSL, GPV, DT, 4, false, 4, false, false, 256>, p, grid, block, lds, stream)
#define FQ_D256_BS(BSL)                           \
    do {                                          \
        if (p.G <= 4) { FQ_D256_GP(BSL, 4); }     \
        else if (p.G <= 8) { FQ_D256_GP(BSL, 8); } \
        else { FQ_D256_GP(BSL, 16); }             \
    } while (0)
    if (BS == 8) FQ_D256_BS(3);
    else if (BS == 16) FQ_D256_BS(4);
    else FQ_D256_BS(5);
#undef FQ_D256_BS
#undef FQ_D256_GP
}

// head_dim 256 with 2 KV heads or 1 on pages of 16 or 32 tokens: rows of 2 or 4 tokens (4 halves of heads or 2 a token).
inline bool staged_d256_linear_applies(int D, int H_KV, int block_size, const DecodeVariant& v) {
    return D == 256 && (H_KV == 1 || H_KV == 2) && block_size >= 16 && !v.direct && v.copy_waves == 4;
}
template <int DT>
int launch_staged_d256_linear(const DecodeParams& p, int S, int rows_per_page, hipStream_t stream) {
    // two tiles of 32 rows (1056 bytes every 1072) and the patch through which the halves of a head exchange their scores
    const size_t lds = 2 * 32 * 1072 + 8 * 2 * kWave * sizeof(float4v);
    const dim3 grid(S, p.num_splits, 1), block(512 + 64 * 4);
#define FQ_D256_FEW(BSL, MULTIV)                                                                                                          \
    do {                                                                                                                                  \
        if (p.G <= 4) return launch_with_lds(paged_decode_staged_kernel<BSL, 4, DT, 4, false, 4, MULTIV, false, 256>, p, grid, block, lds, stream);  \
        if (p.G <= 8) return launch_with_lds(paged_decode_staged_kernel<BSL, 8, DT, 4, false, 4, MULTIV, false, 256>, p, grid, block, lds, stream);  \
        return launch_with_lds(paged_decode_staged_kernel<BSL, 16, DT, 4, false, 4, MULTIV, false, 256>, p, grid, block, lds, stream);    \
    } while (0)
    if (p.H_KV == 2) {
        if (rows_per_page == 8) FQ_D256_FEW(3, 4);
        else FQ_D256_FEW(4, 4);
    } else {
        if (rows_per_page == 4) FQ_D256_FEW(2, 2);
        else FQ_D256_FEW(3, 2);
    }
#undef FQ_D256_FEW
}

template <int D, int DT>
int launch_partials(const DecodeParams& p, int S, int BS, hipStream_t stream, const DecodeVariant& var) {
    if constexpr (D == 256) {
        if (p.new_key == nullptr && p.rotation == nullptr && staged_d256_linear_applies(D, p.H_KV, BS, var)) {
            DecodeParams ps = p;
            ps.balance_slots = staged_balance_slots(S, p.num_splits);
            return launch_staged_d256_linear<DT>(ps, S, BS * p.H_KV / 4, stream);
        }
        if (p.new_key == nullptr && p.rotation == nullptr && staged_d256_applies(D, p.H_KV, var)) {
            const int64_t max_ctx = int64_t(p.max_blocks) * BS;
            const int64_t chunk = (((max_ctx + p.num_splits - 1) / p.num_splits) + 63) & ~int64_t(63);
            DecodeParams ps = p;
            const int groups = p.H_KV / 4;
            ps.balance_slots = staged_balance_slots(S, p.num_splits * groups);
            if (ps.balance_slots > 0) ps.balance_slots = ps.balance_slots / groups > 0 ? ps.balance_slots / groups : 1;
            const bool wide = chunk / BS > 64 || ps.balance_slots > 0 || (p.max_blocks > 64 && p.max_blocks <= 256);
            return launch_staged_d256<DT>(ps, S, BS, wide, stream);
        }
    }
    if constexpr (D == 64) {
        const bool d64_half = staged_d64_half_applies(D, p.H_KV, p.G, BS, var);
        if (d64_half || (p.new_key == nullptr && staged_d64_full_applies(D, p.H_KV, p.G, var))) {
            const int rows_per_page = d64_half ? BS * p.H_KV / 16 : BS;
            const int64_t max_rows = int64_t(p.max_blocks) * rows_per_page;
            const int64_t chunk_rows = (((max_rows + p.num_splits - 1) / p.num_splits) + 63) & ~int64_t(63);
            DecodeParams ps = p;
            ps.G = 2 * p.G;                 // query heads of a pair of KV heads
            const int groups = d64_half ? 1 : p.H_KV / 16;
            ps.balance_slots = staged_balance_slots(S, p.num_splits * groups);
            if (ps.balance_slots > 0) ps.balance_slots = ps.balance_slots / groups > 0 ? ps.balance_slots / groups : 1;
            const bool wide_rows = chunk_rows / rows_per_page > 64 || ps.balance_slots > 0 || (p.max_blocks > 64 && p.max_blocks <= 256);
            return launch_staged_d64<DT>(ps, S, rows_per_page, wide_rows, d64_half, stream);
        }
    }
    if (staged_linear_applies(D, p.H_KV, BS, var)) {     // (one partial per split: also for callers that bring their own partial buffers)
        const int rows_per_page = BS * p.H_KV / 8;
        DecodeParams ps = p;
        ps.balance_slots = staged_balance_slots(S, p.num_splits);
        return launch_staged_linear<DT>(ps, S, rows_per_page, stream);
    }
    // pages a split can span: its tokens are ceil(max_ctx / splits) rounded up to a tile
    const int64_t max_ctx = int64_t(p.max_blocks) * BS;
    const int64_t chunk = (((max_ctx + p.num_splits - 1) / p.num_splits) + 63) & ~int64_t(63);
    const bool wide = chunk / BS > 64;   // begin is a multiple of 64 tokens, hence page aligned

    // four page-id registers also when they can hold the whole block-table row
    if (staged_applies(D, p.H_KV, var)) {
        DecodeParams ps = p;
        // every group of 8 heads is a slice of the grid with the same (sequence, split) pairs
        const int groups = p.H_KV / 8;
        ps.balance_slots = staged_balance_slots(S, p.num_splits * groups);
        if (ps.balance_slots > 0) ps.balance_slots = ps.balance_slots / groups > 0 ? ps.balance_slots / groups : 1;
        // a chosen chunk may span up to 256 pages: four page-id registers
        if (var.ring && p.new_key != nullptr) return FQ_ERR_LAUNCH;
        if (var.ring)
            return launch_ring(ps, S, BS, wide || ps.balance_slots > 0 || (p.max_blocks > 64 && p.max_blocks <= 256), DT, stream);
        return launch_staged_any<DT, false>(ps, S, BS, wide || ps.balance_slots > 0 || (p.max_blocks > 64 && p.max_blocks <= 256),
                                            stream, var.copy_waves, p.new_key != nullptr);
    }
    if (p.new_key != nullptr) return FQ_ERR_LAUNCH;     // only the staged kernel stores the new token

    const int max_waves = D == 256 ? 4 : 8;
    // 1 or 2 KV heads: a full workgroup, its wavefronts beyond the heads on the next splits (measured on 8 x 32768
    // tokens with 2 KV heads: 71 -> 57 us; with 4 heads on 8-token pages, the one case that reaches this kernel, it
    // was slower)
    const bool pack_splits = p.H_KV <= 2 && p.num_splits > 1;
    const int waves = pack_splits ? max_waves : (p.H_KV < max_waves ? p.H_KV : max_waves);
    DecodeParams pk = p;
    pk.heads_per_wg = pack_splits ? p.H_KV : waves;
    const int splits_per_wg = waves / pk.heads_per_wg;
    const dim3 grid((p.num_splits + splits_per_wg - 1) / splits_per_wg, S, (p.H_KV + pk.heads_per_wg - 1) / pk.heads_per_wg),
        block(64 * waves);
    const size_t lds = p.two_tables ? size_t(kLutWords) * sizeof(uint32_t) : 0;   // the K table is static
#define FQ_DECODE_GP(BSL, GPV)                                                                  \
    return wide ? launch_with_lds(paged_decode_kernel<D, BSL, GPV, DT, 4>, pk, grid, block, lds, stream) \
                : launch_with_lds(paged_decode_kernel<D, BSL, GPV, DT, 1>, pk, grid, block, lds, stream)
#define FQ_DECODE_BS(BSL)                             \
    do {                                              \
        if (p.G <= 4) { FQ_DECODE_GP(BSL, 4); }       \
        else if (p.G <= 8) { FQ_DECODE_GP(BSL, 8); }  \
        else { FQ_DECODE_GP(BSL, 16); }               \
    } while (0)
    switch (BS) {
        case 8: FQ_DECODE_BS(3); break;
        case 16: FQ_DECODE_BS(4); break;
        default: FQ_DECODE_BS(5); break;
    }
#undef FQ_DECODE_BS
#undef FQ_DECODE_GP
    return fq_host::check_launch();
}

template <int DT>
int launch_rotate(const void* q, const float* R, int col_major, void* q_rot, int S, int H_Q, int D, hipStream_t stream) {
    const int64_t rows = int64_t(S) * H_Q;
    // as many workgroups per group of 16 rows as it takes to fill the chip, at most one per round of column blocks
    const int64_t row_groups = (rows + kRotRows - 1) / kRotRows;
    const int rounds = D / 64;
    int ysplit = int((fq_host::device_cu_count() + row_groups - 1) / row_groups);
    ysplit = ysplit < 1 ? 1 : (ysplit > rounds ? rounds : ysplit);
    const dim3 grid(static_cast<unsigned>(row_groups), static_cast<unsigned>(ysplit)), block(256);
    const uint16_t* src = reinterpret_cast<const uint16_t*>(q);
    uint16_t* dst = reinterpret_cast<uint16_t*>(q_rot);
    switch (D) {
        case 64: hipLaunchKernelGGL((rotate_q_kernel<64, DT>), grid, block, 0, stream, src, R, dst, rows, col_major); break;
        case 128: hipLaunchKernelGGL((rotate_q_kernel<128, DT>), grid, block, 0, stream, src, R, dst, rows, col_major); break;
        default: hipLaunchKernelGGL((rotate_q_kernel<256, DT>), grid, block, 0, stream, src, R, dst, rows, col_major); break;
    }
    return fq_host::check_launch();
}

template <int DT>
int launch_reduce(const float* acc, const float* m, const float* l, const float* R, int col_major, void* out, int S, int H_Q,
                  int D, int NS, hipStream_t stream) {
    const int64_t rows = int64_t(S) * H_Q;
    // Rows per workgroup: as few as it takes to put a workgroup on every CU, at most 16.  The rows of a
    // decode step are few (1024 at 32 sequences x 32 heads) and the kernel is a chain of latencies
    // (partials, combine, rotate, store), so what counts is how short that chain is per workgroup.
    const int cus = fq_host::device_cu_count();
    const int rw_opt = fq_host::option(FQ_OPT_REDUCE_ROWS);
    int rw = rows <= 4 * int64_t(cus) ? 4 : (rows <= 8 * int64_t(cus) ? 8 : 16);
    if (rw_opt == 4 || rw_opt == 8 || rw_opt == 16) rw = rw_opt;
    // head_dim 256: four workgroups share the columns of a row group, 16 rows a group while that fills the chip
    constexpr int kColumnSplit256 = 4;
    if (D == 256) rw = (rw_opt == 4) ? 4 : 8;       // (a thread stages at most eight coordinates of a row; measured: 8 rows
                                                    // x 4 column groups 79 us per step of 32 x 4096 tokens, 4 rows 81 us)
    const dim3 grid(unsigned((rows + rw - 1) / rw), D == 256 ? kColumnSplit256 : 1), block(256);
    uint16_t* dst = reinterpret_cast<uint16_t*>(out);
#define FQ_REDUCE(DD, RWV) \
    hipLaunchKernelGGL((reduce_rotate_kernel<DD, DT, RWV, (DD == 256 ? kColumnSplit256 : 1)>), grid, block, 0, stream, acc, m, l, R, dst, rows, NS, col_major)
#define FQ_REDUCE_D(DD)                       \
    do {                                      \
        if (rw == 4) FQ_REDUCE(DD, 4);        \
        else if (rw == 8) FQ_REDUCE(DD, 8);   \
        else FQ_REDUCE(DD, 16);               \
    } while (0)
    switch (D) {
        case 64: FQ_REDUCE_D(64); break;
        case 128: FQ_REDUCE_D(128); break;
        default:
            if (rw == 4) FQ_REDUCE(256, 4);
            else FQ_REDUCE(256, 8);
            break;
    }
#undef FQ_REDUCE_D
#undef FQ_REDUCE
    return fq_host::check_launch();
}

int effective_splits(int num_splits, int num_seqs, int H_KV, int D, int block_size, int max_blocks_per_seq);

inline int check_decode_shape(int num_seqs, int H_Q, int H_KV, int D, int block_size, int max_blocks_per_seq,
                              int64_t num_blocks, int dtype, int num_splits) {
    if (num_seqs < 0 || H_Q <= 0 || H_KV <= 0 || max_blocks_per_seq <= 0 || num_blocks <= 0 || num_splits < 0)
        return FQ_ERR_BAD_SHAPE;
    if (H_Q % H_KV != 0 || H_Q / H_KV > 16) return FQ_ERR_BAD_SHAPE;
    if (num_blocks > 0x7fffffffLL || num_seqs > 65535 || (H_KV + 7) / 8 > 65535 || num_splits > 65535)
        return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (block_size != 8 && block_size != 16 && block_size != 32) return FQ_ERR_UNSUPPORTED_BLOCK;
    if (dtype != FQ_F16 && dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    return FQ_OK;
}

}  // namespace fq

namespace fq_host {
int device_cu_count();
bool lds_limit_raised(const void* kernel, size_t bytes) {
    static std::mutex mu;
    static std::map<std::pair<const void*, int>, size_t> done;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) dev = 0;
    std::lock_guard<std::mutex> lock(mu);
    auto it = done.find({kernel, dev});
    if (it != done.end() && it->second >= bytes) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes)) != hipSuccess) {
        note_hip_error(hipGetLastError());
        return false;
    }
    done[{kernel, dev}] = bytes;
    return true;
}
}

// A split keeps its page ids in at most 4 registers of 64 lanes: it may span at most
// 256 pages, which bounds the split count from below for long contexts.
extern "C" int fq_paged_decode_min_splits(int block_size, int max_blocks_per_seq) {
    if (block_size <= 0 || max_blocks_per_seq <= 0) return 1;
    const int64_t max_ctx = int64_t(block_size) * max_blocks_per_seq;
    const int64_t cap = 256 * int64_t(block_size);      // tokens per split, a multiple of 64
    const int64_t ns = (max_ctx + cap - 1) / cap;
    return int(ns < 1 ? 1 : ns);
}

namespace fq {
int auto_splits(int num_seqs, int H_KV, int D, int block_size, int max_blocks_per_seq) {
    if (num_seqs <= 0 || H_KV <= 0 || block_size <= 0 || max_blocks_per_seq <= 0) return 1;
    const int64_t max_ctx = int64_t(block_size) * max_blocks_per_seq;
    const int64_t tiles = (max_ctx + 63) / 64;
    // one round of workgroups over the chip (8 wavefronts per CU, one wavefront per sequence,
    // KV head and split) ...
    const int64_t target_waves = int64_t(fq_host::device_cu_count()) * 8;
    // (4 KV heads run as 8: the staged kernel reads their tokens in pairs; 1 and 2 of dimension 128 likewise, in
    // rows of 8 and 4 tokens; `rows_of_tokens`: the forms that count their chunks in such rows)
    const bool rows_of_tokens = block_size >= 16 && ((D == 128 && (H_KV == 1 || H_KV == 2 || H_KV == 4)) ||
                                                     (D == 64 && (H_KV == 2 || H_KV == 4)) ||
                                                     (D == 256 && (H_KV == 1 || H_KV == 2)));
    const int64_t tokens_per_row = rows_of_tokens ? (D == 128 ? 8 : D == 64 ? 16 : 4) / H_KV : 1;
    int64_t heads = (H_KV == 4 || rows_of_tokens) ? 8 : H_KV;
    // (a workgroup of the staged kernel has 8 wavefronts whatever they serve: a KV head of 256 coordinates takes two
    // of them, a pair of KV heads of 64 coordinates one; measured on 32 x 4096 tokens: head_dim 256 with 8 KV heads
    // 87 us at 8 splits, 82 at 4; head_dim 64 with 16 KV heads 54 us at 4 splits, 37 at 8)
    if (D == 256 && H_KV % 4 == 0) heads = 2 * int64_t(H_KV);
    if (D == 64 && H_KV % 16 == 0) heads = H_KV / 2;
    const int64_t one_round = (target_waves + int64_t(num_seqs) * heads - 1) / (int64_t(num_seqs) * heads);
    // ... and twice that when the contexts are long enough for splits of 1024 tokens: the lengths
    // of the sequences are not known here, a ragged batch leaves many splits empty, and the
    // kernel can merge splits (it sizes its chunks from the actual lengths) but not divide them
    // (rows of tokens: chunks of 1024 rows, not tokens)
    const int64_t long_chunks = max_ctx / (1024 * tokens_per_row);
    int64_t ns = 2 * one_round < long_chunks ? 2 * one_round : long_chunks;
    if (ns < one_round) ns = one_round;
    // Where fewer than 8 KV heads run the direct kernel, its workgroups are as small as the head count: a
    // round over the chip would cut a short context into chunks that cost more to launch and combine
    // than to read (measured on 32 x 4096 tokens: 1 KV head 85 us at 64 splits, 37 us at 16).
    const bool staged_form = rows_of_tokens || (D == 256 && H_KV % 4 == 0) || (D == 64 && H_KV == 8 && block_size >= 16);
    if (H_KV < 8 && !staged_form && ns > max_ctx / 256) ns = max_ctx / 256;
    // (a chunk is at least 64 rows)
    if (rows_of_tokens && ns > max_ctx / (64 * tokens_per_row)) ns = max_ctx / (64 * tokens_per_row);
    if (ns > tiles) ns = tiles;
    // Beyond 128 splits the combine step (one pass over the maxima per 64 splits, one partial row
    // per split) costs more than the shorter chunks save (measured on 1 x 32768 tokens, 8 KV
    // heads: 44.5 us at 64 splits, 44.7 at 128, 58.7 at 256).
    if (ns > 128) ns = 128;
    const int64_t floor_ns = fq_paged_decode_min_splits(block_size, max_blocks_per_seq);
    if (ns < floor_ns) ns = floor_ns;
    if (ns < 1) ns = 1;
    return int(ns);
}
}  // namespace fq

// (for head_dim 128; the other head dimensions differ for 1 and 2 KV heads)
extern "C" int fq_paged_decode_auto_splits(int num_seqs, int H_KV, int block_size, int max_blocks_per_seq) {
    return fq::auto_splits(num_seqs, H_KV, 128, block_size, max_blocks_per_seq);
}

int fq::effective_splits(int num_splits, int num_seqs, int H_KV, int D, int block_size, int max_blocks_per_seq) {
    if (num_splits <= 0) return auto_splits(num_seqs, H_KV, D, block_size, max_blocks_per_seq);
    const int floor_ns = fq_paged_decode_min_splits(block_size, max_blocks_per_seq);
    return num_splits < floor_ns ? floor_ns : num_splits;
}

extern "C" size_t fq_paged_decode_workspace_bytes(int num_seqs, int H_Q, int H_KV, int D, int block_size,
                                                  int max_blocks_per_seq, int num_splits) {
    if (num_seqs <= 0 || H_Q <= 0 || H_KV <= 0 || D <= 0) return 0;
    num_splits = fq::effective_splits(num_splits, num_seqs, H_KV, D, block_size, max_blocks_per_seq);
    return fq::workspace_layout(num_seqs, H_Q, D, num_splits).total;
}

extern "C" int fq_rotate_query(const void* q, const float* rotation, int rotation_col_major, void* q_rot, int64_t num_seqs, int H_Q,
                               int D, int dtype, void* stream) {
    using namespace fq;
    if (num_seqs < 0 || num_seqs > 65535 || H_Q <= 0) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (dtype != FQ_F16 && dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (num_seqs == 0) return FQ_OK;
    if (!q || !rotation || !q_rot) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(rotation, 16) || !fq_host::aligned(q, 16) || !fq_host::aligned(q_rot, 2))
        return FQ_ERR_MISALIGNED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dtype == FQ_F16 ? launch_rotate<FQ_F16>(q, rotation, rotation_col_major, q_rot, int(num_seqs), H_Q, D, s)
                           : launch_rotate<FQ_BF16>(q, rotation, rotation_col_major, q_rot, int(num_seqs), H_Q, D, s);
}

namespace fq {
// Partials of the split-K decode.  `rotation` may be non-NULL only when the staged kernel
// applies: it then rotates the (un-rotated) query itself.
int decode_partials(const void* q, const float* rotation, int rotation_col_major, const uint8_t* kv_cache, const int32_t* block_table,
                    const int32_t* seq_lens, const float* centroids_k, const float* centroids_v, float* partial_acc,
                    float* partial_m, float* partial_l, int num_seqs, int H_Q, int H_KV, int D, int block_size,
                    int max_blocks_per_seq, int64_t num_blocks, float sm_scale, int dtype, int num_splits,
                    void* stream, const DecodeVariant& var, const NewToken* token = nullptr) {
    const int bad = check_decode_shape(num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq, num_blocks, dtype,
                                       num_splits);
    if (bad != FQ_OK) return bad;
    if (num_splits < fq_paged_decode_min_splits(block_size, max_blocks_per_seq)) return FQ_ERR_BAD_SHAPE;
    if (num_seqs == 0) return FQ_OK;
    if (!q || !kv_cache || !block_table || !seq_lens || !centroids_k || !centroids_v || !partial_acc ||
        !partial_m || !partial_l)
        return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(q, 16) || !fq_host::aligned(kv_cache, 16) || !fq_host::aligned(partial_acc, 16) ||
        (rotation && !fq_host::aligned(rotation, 16)))
        return FQ_ERR_MISALIGNED;
    DecodeParams p;
    p.q_rot = q; p.rotation = rotation; p.sketch = nullptr; p.rot_col_major = rotation_col_major; p.cache = kv_cache; p.block_table = block_table; p.seq_lens = seq_lens;
    p.centroids_k = centroids_k; p.centroids_v = centroids_v;
    p.part_acc = partial_acc; p.part_m = partial_m; p.part_l = partial_l;
    p.H_Q = H_Q; p.H_KV = H_KV; p.G = H_Q / H_KV; p.max_blocks = max_blocks_per_seq;
    p.num_blocks = int(num_blocks); p.num_splits = num_splits;
    p.two_tables = centroids_k != centroids_v ? 1 : 0;
    p.scale_log2e = sm_scale * kLog2e;
    p.balance_slots = 0;
    p.heads_per_wg = 0;
    p.spin_limit = fq_host::option(FQ_OPT_DECODE_TINY_SPIN) != 0 ? 2 : (1 << 20);
    p.cache_rw = token ? token->cache : nullptr;
    p.new_key = token ? token->key : nullptr;
    p.new_value = token ? token->value : nullptr;
    p.new_slots = token ? token->slots : nullptr;
    p.boundaries = token ? token->boundaries : nullptr;
    p.num_slots = num_blocks * block_size;
    hipStream_t s = static_cast<hipStream_t>(stream);
#define FQ_DECODE_D(DD)                                                                 \
    case DD:                                                                            \
        return dtype == FQ_F16 ? launch_partials<DD, FQ_F16>(p, num_seqs, block_size, s, var) \
                               : launch_partials<DD, FQ_BF16>(p, num_seqs, block_size, s, var);
    switch (D) {
        FQ_DECODE_D(64)
        FQ_DECODE_D(128)
        FQ_DECODE_D(256)
        default: return FQ_ERR_UNSUPPORTED_DIM;
    }
#undef FQ_DECODE_D
}
}  // namespace fq

extern "C" int fq_paged_decode_fault_count(unsigned int* count) {
    if (!count) return FQ_ERR_NULL_POINTER;
    const hipError_t e = hipMemcpyFromSymbol(count, HIP_SYMBOL(fq::g_decode_faults), sizeof(unsigned int));
    if (e != hipSuccess) {
        fq_host::note_hip_error(e);
        return FQ_ERR_LAUNCH;
    }
    return FQ_OK;
}

extern "C" int fq_paged_decode_fuses_rotation(int D, int H_KV, int shared_codebook) {
    (void)shared_codebook;   // both codebooks fit the kernel's table
    return fq::staged_applies(D, H_KV, fq::read_decode_variant()) ? 1 : 0;
}

extern "C" int fq_paged_tq4_decode(const void* q, const float* rotation, int rotation_col_major,
                                   const uint8_t* kv_cache, const int32_t* block_table, const int32_t* seq_lens,
                                   const float* centroids_k, const float* centroids_v, float* partial_acc,
                                   float* partial_m, float* partial_l, int num_seqs, int H_Q, int H_KV, int D,
                                   int block_size, int max_blocks_per_seq, int64_t num_blocks, float sm_scale,
                                   int dtype, int num_splits, void* stream) {
    const fq::DecodeVariant var = fq::read_decode_variant();      // one reading of the switches per call
    if (rotation && !fq::staged_applies(D, H_KV, var)) return FQ_ERR_BAD_SHAPE;
    return fq::decode_partials(q, rotation, rotation_col_major, kv_cache, block_table, seq_lens, centroids_k,
                               centroids_v, partial_acc, partial_m, partial_l, num_seqs, H_Q, H_KV, D, block_size,
                               max_blocks_per_seq, num_blocks, sm_scale, dtype, num_splits, stream, var);
}

extern "C" int fq_split_k_reduce(const float* partial_acc, const float* partial_m, const float* partial_l,
                                 const float* rotation, int rotation_col_major, void* out, int num_seqs, int H_Q, int D, int dtype,
                                 int num_splits, void* stream) {
    using namespace fq;
    if (num_seqs < 0 || num_seqs > 65535 || H_Q <= 0 || num_splits < 1) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (dtype != FQ_F16 && dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (num_seqs == 0) return FQ_OK;
    if (!partial_acc || !partial_m || !partial_l || !out) return FQ_ERR_NULL_POINTER;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return dtype == FQ_F16
               ? launch_reduce<FQ_F16>(partial_acc, partial_m, partial_l, rotation, rotation_col_major, out, num_seqs, H_Q, D, num_splits, s)
               : launch_reduce<FQ_BF16>(partial_acc, partial_m, partial_l, rotation, rotation_col_major, out, num_seqs, H_Q, D, num_splits, s);
}

namespace fq {
// fq_split_k_paged_decode for one reading `var` of the switches; `token`: the staged kernel (which must be
// the one that `var` selects for this shape) also stores the step's new token.
int split_k_paged_decode_impl(const void* q, const uint8_t* kv_cache, const int32_t* block_table,
                              const int32_t* seq_lens, const float* centroids_k,
                              const float* centroids_v, const float* rotation, int rotation_col_major, void* out,
                              int num_seqs, int H_Q, int H_KV, int D, int block_size,
                              int max_blocks_per_seq, int64_t num_blocks, float sm_scale, int dtype,
                              int num_splits, void* workspace, size_t workspace_bytes, void* stream,
                              const DecodeVariant& var, const NewToken* token) {
    const int bad = check_decode_shape(num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq, num_blocks, dtype,
                                       num_splits);
    if (bad != FQ_OK) return bad;
    if (num_seqs == 0) return FQ_OK;
    if (!q || !out) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(q, 16) || !fq_host::aligned(out, 16)) return FQ_ERR_MISALIGNED;
    num_splits = effective_splits(num_splits, num_seqs, H_KV, D, block_size, max_blocks_per_seq);
    const int G = H_Q / H_KV;
    // the forms of the staged kernel on rows of several tokens (they too write one partial per split)
    const bool half = staged_linear_applies(D, H_KV, block_size, var) || staged_d64_half_applies(D, H_KV, G, block_size, var);
    const int num_partials = num_splits;
    const WorkspaceLayout w = workspace_layout(num_seqs, H_Q, D, num_partials);
    if (!workspace || workspace_bytes < w.total) return FQ_ERR_WORKSPACE;
    if (!fq_host::aligned(workspace, 256)) return FQ_ERR_MISALIGNED;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    float* acc = reinterpret_cast<float*>(ws + w.acc);
    float* m = reinterpret_cast<float*>(ws + w.m);
    float* l = reinterpret_cast<float*>(ws + w.l);
    const void* q_in = q;
    const float* fused_rotation = nullptr;
    if (rotation) {
        if (centroids_k && (half || staged_applies(D, H_KV, var) || (token == nullptr && staged_d64_full_applies(D, H_KV, G, var)))) {
            fused_rotation = rotation;       // the staged kernel rotates the query in its prologue
        } else {
            const int st = fq_rotate_query(q, rotation, rotation_col_major, ws + w.qrot, num_seqs, H_Q, D, dtype, stream);
            if (st != FQ_OK) return st;
            q_in = ws + w.qrot;
        }
    }
    int st = decode_partials(q_in, fused_rotation, rotation_col_major, kv_cache, block_table, seq_lens, centroids_k, centroids_v, acc, m,
                             l, num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq, num_blocks, sm_scale, dtype,
                             num_splits, stream, var, token);
    if (st != FQ_OK) return st;
    return fq_split_k_reduce(acc, m, l, rotation, rotation_col_major, out, num_seqs, H_Q, D, dtype, num_partials, stream);
}
}  // namespace fq

extern "C" int fq_split_k_paged_decode(const void* q, const uint8_t* kv_cache, const int32_t* block_table,
                                       const int32_t* seq_lens, const float* centroids_k,
                                       const float* centroids_v, const float* rotation, int rotation_col_major, void* out,
                                       int num_seqs, int H_Q, int H_KV, int D, int block_size,
                                       int max_blocks_per_seq, int64_t num_blocks, float sm_scale, int dtype,
                                       int num_splits, void* workspace, size_t workspace_bytes, void* stream) {
    // One reading of the kernel-variant switches for the whole call: the kernel choice, the number of
    // partials it writes, the workspace layout and what the combine kernel merges all follow from it.
    return fq::split_k_paged_decode_impl(q, kv_cache, block_table, seq_lens, centroids_k, centroids_v, rotation,
                                         rotation_col_major, out, num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq,
                                         num_blocks, sm_scale, dtype, num_splits, workspace, workspace_bytes, stream,
                                         fq::read_decode_variant(), nullptr);
}

// One serving step: the new token of every sequence compressed into its cache row, then the decode over
// the cache that holds it (src/flashquant/vllm/impl.py:362-394).  One launch fewer where the staged
// kernel with copy wavefronts runs (KV heads of dimension 128 in groups of 8, a rotation matrix given):
// the workgroup whose split ends with a sequence's last token compresses and stores that token itself.
extern "C" int fq_tq4_store_and_decode(const void* key, const void* value, const int64_t* slot_mapping,
                                       const float* rot_T_even, const float* rot_T_odd, const float* boundaries,
                                       const void* q, uint8_t* kv_cache, const int32_t* block_table,
                                       const int32_t* seq_lens, const float* centroids_k, const float* centroids_v,
                                       const float* rotation, int rotation_col_major, void* out, int num_seqs,
                                       int H_Q, int H_KV, int D, int block_size, int max_blocks_per_seq,
                                       int64_t num_blocks, float sm_scale, int dtype, int num_splits,
                                       void* workspace, size_t workspace_bytes, void* stream) {
    using namespace fq;
    const int bad = check_decode_shape(num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq, num_blocks, dtype,
                                       num_splits);
    if (bad != FQ_OK) return bad;
    if (num_seqs == 0) return FQ_OK;
    if (!key || !value || !slot_mapping || !rot_T_even || !rot_T_odd || !boundaries || !rotation || !kv_cache)
        return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(key, 16) || !fq_host::aligned(value, 16) || !fq_host::aligned(slot_mapping, 8) ||
        !fq_host::aligned(kv_cache, 16) || !fq_host::aligned(boundaries, 4))
        return FQ_ERR_MISALIGNED;
    const DecodeVariant var = read_decode_variant();
    const bool in_launch = centroids_k && var.copy_waves == 4 &&
                           ((staged_applies(D, H_KV, var) && !var.ring) || staged_linear_applies(D, H_KV, block_size, var) ||
                            staged_d64_half_applies(D, H_KV, H_Q / H_KV, block_size, var));
    const NewToken token{key, value, slot_mapping, boundaries, kv_cache};
    if (!in_launch) {
        const int st = fq_tq4_compress_store(key, value, dtype, rot_T_even, rot_T_odd, boundaries, kv_cache, slot_mapping,
                                             num_seqs, num_seqs, H_KV, D, num_blocks * block_size, stream);
        if (st != FQ_OK) return st;
    }
    return split_k_paged_decode_impl(q, kv_cache, block_table, seq_lens, centroids_k, centroids_v, rotation,
                                     rotation_col_major, out, num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq,
                                     num_blocks, sm_scale, dtype, num_splits, workspace, workspace_bytes, stream, var,
                                     in_launch ? &token : nullptr);
}

// ---------------------------------------------------------------------------------------
// The same decode for callers that cannot allocate (HIP graph capture, serving loops whose
// harness forbids hipMalloc): the split partials and the rotated query live in a file-scope
// device array instead of a caller workspace.  Every GPU the library runs on holds its own
// copy of the array until the process ends; the host keeps each copy's address per device.
// ---------------------------------------------------------------------------------------
namespace fq {
constexpr size_t kStaticScratchBytes = size_t(FQ_STATIC_SCRATCH_BYTES);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
}  // namespace fq

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device.  The array's name is a host-side handle,
// not an address a kernel can use: the address comes from the runtime, once per device.
int static_scratch_address(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) {
        fq_host::note_hip_error(e);
        return FQ_ERR_LAUNCH;
    }
    if (dev < 0 || dev >= kMaxDevices) return FQ_ERR_BAD_SHAPE;
    std::lock_guard<std::mutex> lock(g_scratch_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(fq::scratch));
        if (e != hipSuccess || p == nullptr) {
            fq_host::note_hip_error(e);
            return FQ_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return FQ_OK;
}
}  // namespace

extern "C" size_t fq_static_scratch_bytes(void) { return fq::kStaticScratchBytes; }

extern "C" int fq_split_k_paged_decode_static(const void* q, const uint8_t* kv_cache, const int32_t* block_table,
                                              const int32_t* seq_lens, const float* centroids_k,
                                              const float* centroids_v, const float* rotation,
                                              int rotation_col_major, void* out, int num_seqs, int H_Q, int H_KV,
                                              int D, int block_size, int max_blocks_per_seq, int64_t num_blocks,
                                              float sm_scale, int dtype, int num_splits, void* stream) {
    using namespace fq;
    const int bad = check_decode_shape(num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq, num_blocks, dtype,
                                       num_splits);
    if (bad != FQ_OK) return bad;
    if (num_seqs == 0) return FQ_OK;
    const int ns = effective_splits(num_splits, num_seqs, H_KV, D, block_size, max_blocks_per_seq);
    // the partials of this launch must fit the array: a larger problem is refused, not truncated
    const int num_partials = ns;
    if (workspace_layout(num_seqs, H_Q, D, num_partials).total > kStaticScratchBytes) return FQ_ERR_WORKSPACE;
    void* ws = nullptr;
    const int st = static_scratch_address(&ws);
    if (st != FQ_OK) return st;
    // Nothing in the array has to start at zero: every (sequence, head, split) slot of the maxima
    // and denominators is written by the decode kernel of this call (an empty split writes
    // m = -inf), and the combine kernel ignores the accumulators of empty splits.
    return fq_split_k_paged_decode(q, kv_cache, block_table, seq_lens, centroids_k, centroids_v, rotation,
                                   rotation_col_major, out, num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq,
                                   num_blocks, sm_scale, dtype, ns, ws, kStaticScratchBytes, stream);
}

// TurboQuantProd pages: 3-bit keys with a sign-sketch correction of the scores, TQ4 values.
extern "C" int fq_prod_paged_decode(const void* q, const uint8_t* kv_cache, const int32_t* block_table,
                                    const int32_t* seq_lens, const float* centroids_k3,
                                    const float* centroids_v, const float* rotation, int rotation_col_major,
                                    const float* sketch, void* out, int num_seqs, int H_Q, int H_KV, int D,
                                    int block_size, int max_blocks_per_seq, int64_t num_blocks, float sm_scale,
                                    int dtype, int num_splits, void* workspace, size_t workspace_bytes,
                                    void* stream) {
    using namespace fq;
    const int bad = check_decode_shape(num_seqs, H_Q, H_KV, D, block_size, max_blocks_per_seq, num_blocks, dtype,
                                       num_splits);
    if (bad != FQ_OK) return bad;
    if (D != 128) return FQ_ERR_UNSUPPORTED_DIM;
    // the kernel stages the token rows of 8 KV heads, and the sketched queries of a group of 8 (float32,
    // beside the rotated ones) fit its LDS for up to 8 query heads per KV head
    if (H_KV % 8 != 0 || H_Q / H_KV > 8) return FQ_ERR_BAD_SHAPE;
    if (num_seqs == 0) return FQ_OK;
    if (!q || !out || !kv_cache || !block_table || !seq_lens || !centroids_k3 || !centroids_v || !rotation || !sketch)
        return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(q, 16) || !fq_host::aligned(out, 16) || !fq_host::aligned(kv_cache, 16) ||
        !fq_host::aligned(rotation, 16) || !fq_host::aligned(sketch, 16))
        return FQ_ERR_MISALIGNED;
    num_splits = effective_splits(num_splits, num_seqs, H_KV, D, block_size, max_blocks_per_seq);
    const WorkspaceLayout w = workspace_layout(num_seqs, H_Q, D, num_splits);
    if (!workspace || workspace_bytes < w.total) return FQ_ERR_WORKSPACE;
    if (!fq_host::aligned(workspace, 256)) return FQ_ERR_MISALIGNED;
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    float* acc = reinterpret_cast<float*>(ws + w.acc);
    float* m = reinterpret_cast<float*>(ws + w.m);
    float* l = reinterpret_cast<float*>(ws + w.l);

    DecodeParams p;
    p.q_rot = q; p.rotation = rotation; p.sketch = sketch; p.rot_col_major = rotation_col_major;
    p.cache = kv_cache; p.block_table = block_table; p.seq_lens = seq_lens;
    p.centroids_k = centroids_k3; p.centroids_v = centroids_v;
    p.part_acc = acc; p.part_m = m; p.part_l = l;
    p.H_Q = H_Q; p.H_KV = H_KV; p.G = H_Q / H_KV; p.max_blocks = max_blocks_per_seq;
    p.num_blocks = int(num_blocks); p.num_splits = num_splits;
    p.two_tables = 1;
    p.scale_log2e = sm_scale * kLog2e;
    // every group of 8 heads is a slice of the grid with the same (sequence, split) pairs
    const int groups = H_KV / 8;
    p.balance_slots = staged_balance_slots(num_seqs, num_splits * groups);
    if (p.balance_slots > 0) p.balance_slots = p.balance_slots / groups > 0 ? p.balance_slots / groups : 1;
    p.heads_per_wg = 0;
    p.spin_limit = fq_host::option(FQ_OPT_DECODE_TINY_SPIN) != 0 ? 2 : (1 << 20);
    p.cache_rw = nullptr; p.new_key = nullptr; p.new_value = nullptr; p.new_slots = nullptr; p.boundaries = nullptr;
    p.num_slots = 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int64_t max_ctx = int64_t(max_blocks_per_seq) * block_size;
    const int64_t chunk = (((max_ctx + num_splits - 1) / num_splits) + 63) & ~int64_t(63);
    const bool wide = chunk / block_size > 64 || p.balance_slots > 0 ||
                      (max_blocks_per_seq > 64 && max_blocks_per_seq <= 256);
    const int copy_waves = read_decode_variant().copy_waves;
    const int st = dtype == FQ_F16 ? launch_staged_any<FQ_F16, true>(p, num_seqs, block_size, wide, s, copy_waves)
                                   : launch_staged_any<FQ_BF16, true>(p, num_seqs, block_size, wide, s, copy_waves);
    if (st != FQ_OK) return st;
    return fq_split_k_reduce(acc, m, l, rotation, rotation_col_major, out, num_seqs, H_Q, D, dtype, num_splits, stream);
}
