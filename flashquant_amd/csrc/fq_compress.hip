// TQ4 compress for gfx950.
//
// Per row x (D elements, fp16 or bf16):  n = ||x||_2,  y = (x / (n + 1e-10)) R^T,
// idx_j = #{boundaries < y_j},  byte_j = idx_2j << 4 | idx_2j+1,  norm = n
// (compress_reference, src/flashquant/kernels/cpu_reference.py:39-61).
//
// The rotation is a rows x D x D contraction on the 32x32x16 fp16 MFMA, with
// float32 accumulation.  A plain 16-bit rotation would move about 1 index in
// 200 across a bucket boundary, so the matrix is split R = R_hi + 2^-12 R_lo
// (two fp16 terms, 22 significant bits) and the row is rotated un-normalised:
// the raw fp16/bf16 row, scaled by a power of two so that its largest element
// lies in [1, 2), is exact in fp16 up to elements 2^-24 below the largest, and
// the division by (n + 1e-10) is applied to the float32 accumulators.
//
// Layout.  One workgroup owns the whole matrix in registers: wave w keeps the
// MFMA A operands (R_hi, R_lo rows of its 32 output coordinates, all k) for the
// kernel's lifetime.  Tiles of 64 rows stream through LDS as the B operand
// (row-major fp16, padded rows so that the 128-bit operand reads are
// conflict-free), double buffered against the global loads of the next tile.
// A lane of the accumulator holds one row and 16 consecutive output
// coordinates (the MFMA row index is permuted on the R side to make them
// consecutive), so a lane bucketizes and nibble-packs 8 output bytes without
// any cross-lane traffic.  Bucketize is one LDS lookup in a 64-cell table
// built from the boundaries (base count + the single boundary that can fall in
// the cell; 32 copies of every cell, one per bank) plus one compare; if two
// boundaries share a cell the kernel falls back to the 15-compare scan.

#include "fq_common.hpp"

namespace fq {

template <int D>
struct CompressCfg {
    static constexpr int NK = D / 16;                  // MFMA k-steps
    static constexpr int CB = D / 32;                  // 32-coordinate output blocks
    static constexpr int WAVES = CB < 4 ? 4 : CB;
    static constexpr int THREADS = WAVES * kWave;
    static constexpr int TT = D == 256 ? 32 : 64;      // rows per tile
    static constexpr int TB = TT / 32;                 // 32-row blocks per tile
    static constexpr int TB_STEP = WAVES / CB;         // row blocks handled in parallel
    static constexpr int CPR = D / 8;                  // 16-byte chunks per row
    static constexpr int ROWS_PER_PASS = THREADS / CPR;
    static constexpr int PASSES = TT / ROWS_PER_PASS;
    static constexpr int XS_STRIDE = D * 2 + 16;       // bytes per staged row
    static constexpr int OUT_STRIDE = D / 2 + 8;       // bytes per packed row in LDS
};

constexpr float kLoScale = 1.0f / 4096.0f;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// top 16 bits of a float as bf16 (truncation: the next term of the split takes up the rest)
__device__ __forceinline__ __bf16 bf16_trunc(float f) {
    return __builtin_bit_cast(__bf16, uint16_t(float_to_bits(f) >> 16));
}
// nearest bf16, ties to even (finite inputs)
__device__ __forceinline__ __bf16 bf16_nearest(float f) {
    const uint32_t b = float_to_bits(f);
    return __builtin_bit_cast(__bf16, uint16_t((b + 0x7fffu + ((b >> 16) & 1u)) >> 16));
}
__device__ __forceinline__ float bf16_value(__bf16 h) {
    return bits_to_float(uint32_t(__builtin_bit_cast(uint16_t, h)) << 16);
}

// lane exchange inside the VALU (DPP): CTRL 0xB1 / 0x4E swap lanes inside quads, 0x141 / 0x140
// mirror the 8- / 16-lane rows
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}

// 128 cells over the span of the boundaries, every cell stored 32 times side by side (a cell is a
// 256-byte row of 32 copies of 8 bytes): lane l reads copy l % 32, so the lanes of a half-wave
// always hit different banks whatever cells their values fall in.  A single copy made the
// data-dependent lookups collide (4-5 lanes per bank on average).
//
// The table is the first object of the kernel's LDS block, at LDS address 0: the address of a lane's
// copy of cell c is then (c << 8) | (8 * copy), which v_cvt_pk_u8_f32 builds in one instruction from
// the cell coordinate (float -> integer saturated to 0..255, written into byte 1 of the lane's
// constant 8 * copy).  A value y is looked up by its cell coordinate pos = y / w + offset and compared
// with the cell's boundary as it is (in the cell coordinate values within 3e-8 of the boundary 0 would
// lose their sign, which is all that rows of negligible norm have).  The conversion's rounding is left
// open: a cell answers for the coordinates one cell to either side of its own as well.
constexpr int kBucketCells = 128;
constexpr int kBucketCopies = 32;
struct BucketTable {
    uint2v cell[kBucketCells * kBucketCopies];   // x = threshold bits, y = base count
    float bnd[16];
    float inv_w;
    float offset;
    int slow;
};
typedef __attribute__((address_space(3))) const uint2v lds_cell_t;

// LDS address of an object
template <typename T>
__device__ __forceinline__ uint32_t lds_address(const T* p) {
    return uint32_t(reinterpret_cast<uintptr_t>((__attribute__((address_space(3))) const void*)p));
}

// Builds the cell table from the 15 boundaries (block-wide, ends with a barrier).
__device__ __forceinline__ void build_bucket_table(BucketTable& t, const float* __restrict__ boundaries,
                                                   int tid, int nthreads) {
    if (tid < 15) t.bnd[tid] = boundaries[tid];
    if (tid == 15) t.bnd[15] = __builtin_inff();
    // the one-instruction address needs the table at LDS address 0
    if (tid == 0) t.slow = lds_address(&t.cell[0]) != 0u ? 1 : 0;
    __syncthreads();
    const float b0 = t.bnd[0], b14 = t.bnd[14];
    const float span = b14 - b0;
    // two cells of padding on either side of the outer boundaries
    const float w = span > 0.0f ? span * (1.0f / float(kBucketCells - 4)) : 1.0f;
    const float lo = b0 - 2.0f * w;
    const float inv_w = 1.0f / w, offset = -lo / w;
    for (int c = tid; c < kBucketCells; c += nthreads) {
        // coordinates that may be converted to cell c: [c - 1, c + 2), with a margin for rounding
        const float lo_c = float(c) - 1.01f;
        const float hi_c = float(c) + 2.01f;
        int base = 0, inside = 0;
        float thr = __builtin_inff();
        for (int b = 0; b < 15; ++b) {
            const float v = __builtin_fmaf(t.bnd[b], inv_w, offset);
            if (v < lo_c) {
                ++base;
            } else if (v <= hi_c) {
                ++inside;
                thr = t.bnd[b];
            }
        }
        if (inside > 1 || !(span > 0.0f)) t.slow = 1;
        for (int k = 0; k < kBucketCopies; ++k) t.cell[c * kBucketCopies + k] = uint2v{float_to_bits(thr), uint32_t(base)};
    }
    if (tid == 0) {
        t.inv_w = inv_w;
        t.offset = offset;
    }
    __syncthreads();
}

// `copy8` = 8 * (lane % 32)
__device__ __forceinline__ uint2v bucket_cell(float y, float inv_w, float offset, uint32_t copy8) {
    const float pos = __builtin_fmaf(y, inv_w, offset);
    // the conversion saturates at 0 and 255, the table ends at cell 127; the median also sends a NaN
    // to cell 0 (no boundary lies below a NaN: index 0, as the reference's count gives)
    const float top = __builtin_amdgcn_fmed3f(pos, 0.0f, float(kBucketCells - 1));
    const uint32_t addr = __builtin_amdgcn_cvt_pk_u8_f32(top, 1u, copy8);
    return *reinterpret_cast<lds_cell_t*>(addr);
}
__device__ __forceinline__ uint32_t bucket_fast(float y, float inv_w, float offset, uint32_t copy8) {
    const uint2v e = bucket_cell(y, inv_w, offset, copy8);
    return e.y + (bits_to_float(e.x) < y ? 1u : 0u);
}

__device__ __forceinline__ uint32_t bucket_slow(const BucketTable& t, float y) {
    uint32_t n = 0;
#pragma unroll
    for (int b = 0; b < 15; ++b) n += (t.bnd[b] < y) ? 1u : 0u;
    return n;
}

// MFMA row r of a 32-row block <-> output coordinate (within the block) such
// that accumulator register i of lane half h holds coordinate 16h + i.
__device__ __forceinline__ int mfma_row_to_coord(int r) {
    return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3);
}

// Destination of the fused compress-and-store (the work of _compress_and_store,
// src/flashquant/vllm/impl.py:220-263, in one launch): rows [0, rows_k) come from the key
// tensor and rows [rows_k, 2 rows_k) from the value tensor, row = token * H + head, and each
// lands in the paged cache row of slot_mapping[token]:
// [K idx H*D/2 | K norm H*4 | V idx H*D/2 | V norm H*4] (src/flashquant/vllm/impl.py:132-138).
struct PagedDest {
    const uint4v* x_value;      // (tokens, H, D) values
    uint8_t* cache;             // (num_slots, H*(D+8))
    const int64_t* slots;       // (mapped,) flat slot of each token; negative: not stored
    int64_t rows_k;             // tokens * H
    uint32_t tokens;
    int64_t num_slots;
    int mapped;                 // tokens with a slot
    int H;
    int wide;                   // 16-byte stores are aligned
    // plain (not paged) mode, append into a buffer of larger capacity: input row (o, t), t < append_n,
    // lands in output row o * append_cap + append_pos + t; append_n == 0: output row = input row
    uint32_t append_n;
    int64_t append_cap, append_pos;
};

// NT: bf16 terms of the rotation matrix for bf16 rows (ignored for fp16 rows; three at head_dim 256 means the fp16 route).
// 3: R = t0 + t1 + t2 exactly.  2: t0, t1 rounded to nearest, |R - t0 - t1| <= 2^-18 |R|: the rotated
// coordinates move by about 2e-7 (standard deviation, unit rows of 128 coordinates), which puts about 6
// indices in a million on the other side of a bucket boundary, for two thirds of the matrix instructions.
template <int D, int DT, bool PAGED, int NT>
__global__ __launch_bounds__(CompressCfg<D>::THREADS) void tq4_compress_kernel(
    const uint4v* __restrict__ x, const float* __restrict__ rot_T_even,
    const float* __restrict__ rot_T_odd, const float* __restrict__ boundaries,
    uint8_t* __restrict__ packed, float* __restrict__ norms, int64_t M, int64_t num_tiles, const PagedDest pd) {
    using C = CompressCfg<D>;
    // Rows are grouped by a divisor: in paged mode the H heads of a token, in append mode the append_n
    // new tokens of a (batch, head) pair.  The first row of a tile is row0 = q * divisor + r (Origin,
    // wave-uniform, carried from tile to tile by additions); row0 + i then belongs to group
    // q + (r + i) / divisor, at place (r + i) % divisor.  In paged mode rows_k is a multiple of H, so
    // the same pair serves the rows of both tensors (token counted over keys, then values).
    struct Origin { uint32_t q, r; };
    const uint32_t divisor = PAGED ? uint32_t(pd.H) : (pd.append_n != 0u ? pd.append_n : 1u);
    const float rcp_div = 1.0f / float(divisor);
    auto origin_of = [&](uint32_t first_tile) {
        const uint32_t row0 = first_tile * uint32_t(C::TT);      // the first tiles: below 2^32 rows
        return Origin{row0 / divisor, row0 % divisor};
    };
    const Origin tile_step = origin_of(gridDim.x);
    auto advance = [&](Origin o) {
        o.q += tile_step.q;
        o.r += tile_step.r;
        if (o.r >= divisor) { o.r -= divisor; o.q += 1u; }
        return o;
    };
    // group and place of row i of the tile
    auto locate = [&](Origin o, int i, uint32_t& group, uint32_t& place) {
        const uint32_t t = o.r + uint32_t(i);                       // < divisor + TT
        // t / divisor: (t + 1/2) / divisor lies at least 1 / (2 divisor) away from an integer, far more
        // than the rounding of the float32 product while the divisor is below 2^20; a larger divisor
        // exceeds t at most once
        uint32_t dq = uint32_t(__builtin_fmaf(float(t), rcp_div, 0.5f * rcp_div));
        if (!PAGED && divisor >= (1u << 20)) dq = t >= divisor ? 1u : 0u;
        group = o.q + dq;
        place = t - dq * divisor;
    };
    // paged mode: cache row of row i of the tile, or nullptr when the token has no slot
    auto paged_row = [&](Origin o, int i, int& head, int& is_v) -> uint8_t* {
        uint32_t tok, hd;
        locate(o, i, tok, hd);
        head = int(hd);
        is_v = tok >= pd.tokens ? 1 : 0;
        tok -= is_v ? pd.tokens : 0u;
        if (tok >= uint32_t(pd.mapped)) return nullptr;
        const int64_t slot = pd.slots[tok];
        if (slot < 0 || slot >= pd.num_slots) return nullptr;
        return pd.cache + slot * (int64_t(pd.H) * (D + 8)) + (is_v ? int64_t(pd.H) * (D / 2 + 4) : 0);
    };
    // plain mode appending into a buffer of larger capacity: output row of row i of the tile
    auto appended_row = [&](Origin o, int i) -> int64_t {
        uint32_t outer, t;
        locate(o, i, outer, t);
        return int64_t(outer) * pd.append_cap + pd.append_pos + int64_t(t);
    };
    // head_dim 128 runs a software pipeline (see below) with two packed-row buffers
    constexpr bool kPipe = D == 128;
    constexpr int kOutBytes = C::TT * C::OUT_STRIDE;
    // one LDS block, the bucket table first (its lookups address it from LDS address 0)
    struct Lds {
        BucketTable table;
        __attribute__((aligned(16))) uint8_t xs[2][C::TT * C::XS_STRIDE];
        __attribute__((aligned(16))) uint8_t outs[(kPipe ? 2 : 1) * kOutBytes];
        float inv_s[2][C::TT];
    };
    __shared__ __attribute__((aligned(256))) Lds lds;
    BucketTable& table = lds.table;
    auto& xs = lds.xs;
    auto& outs = lds.outs;
    auto& inv_s = lds.inv_s;

    const int tid = threadIdx.x;
    const int wave = tid / kWave;
    const int lane = tid % kWave;
    const int n32 = lane % 32;   // MFMA row (A side) / tile row (B, C side)
    const int kg = lane / 32;    // k group (A, B side) / coordinate half (C side)
    const int cb = wave % C::CB;
    const int tb0 = wave / C::CB;

    // ---- staging helpers -----------------------------------------------------
    const int chunk = tid % C::CPR;
    const int row_in_pass = tid / C::CPR;
    uint4v pre[C::PASSES];

    // Everything that depends on the tile alone is wave-uniform (scalar registers); a thread adds
    // 32-bit offsets to it.  rows_in(tile): rows of the tile that exist (0..TT).
    auto rows_in = [&](int64_t tile) -> int {
        const int64_t left = M - tile * C::TT;
        return left >= C::TT ? C::TT : (left > 0 ? int(left) : 0);
    };
    auto issue_loads = [&](int64_t tile) {
        const int64_t row0 = tile * C::TT;
        const int live = rows_in(tile);
        const uint4v* base = x + row0 * C::CPR;
        // paged mode: rows [rows_k, 2 rows_k) come from the value tensor; a tile may hold rows of both
        int first_v = C::TT;
        const uint4v* base_v = base;
        if (PAGED) {
            const int64_t k_left = pd.rows_k - row0;
            first_v = k_left >= C::TT ? C::TT : (k_left > 0 ? int(k_left) : 0);
            base_v = reinterpret_cast<const uint4v*>(reinterpret_cast<uintptr_t>(pd.x_value) +
                                                     uintptr_t((row0 - pd.rows_k) * C::CPR * int64_t(sizeof(uint4v))));
        }
        if (!PAGED && live == C::TT) {       // uniform: a whole tile needs no per-row conditions
#pragma unroll
            for (int p = 0; p < C::PASSES; ++p)
                pre[p] = __builtin_nontemporal_load(base + p * C::ROWS_PER_PASS * C::CPR + tid);
            return;
        }
#pragma unroll
        for (int p = 0; p < C::PASSES; ++p) {
            const int r = p * C::ROWS_PER_PASS + row_in_pass;
            const int off = p * C::ROWS_PER_PASS * C::CPR + tid;           // r * CPR + chunk
            const uint4v* src = (PAGED && r >= first_v) ? base_v : base;
            pre[p] = r < live ? __builtin_nontemporal_load(src + off) : uint4v{0, 0, 0, 0};
        }
    };
    // the rows of the first tile are asked for before anything else: they arrive while the matrix rows are
    // fetched and the bucket table is built (a small call is all prologue)
    if (int64_t(blockIdx.x) < num_tiles) issue_loads(blockIdx.x);

    // ---- the rotation rows of this wave, split into two fp16 terms ----------
    // fp16 rows: R = hi + lo / 4096 in fp16.  bf16 rows go to the bf16 MFMA as they are, against
    // R = t0 + t1 (+ t2) in bf16 (3 x 8 bits: the float32 value exactly); bf16 terms keep the
    // float32 exponent range, so the products share one accumulator.
    // (head_dim 256 would need 192 registers for three terms: with three it takes the fp16 route)
    constexpr bool kBf16 = DT == FQ_BF16 && (D <= 128 || NT == 2);
    static_assert(NT == 2 || NT == 3, "two or three bf16 terms");
    half8 a_hi[kBf16 ? 1 : C::NK], a_lo[kBf16 ? 1 : C::NK];
    bf16x8 a_t[kBf16 ? NT : 1][kBf16 ? C::NK : 1];
    // the matrix rows are asked for, the bucket table is built while they arrive, then they are split
    float rr[C::NK][8];
    {
        const int j = 32 * cb + mfma_row_to_coord(n32);
        const float* src = (j & 1) ? rot_T_odd : rot_T_even;
        const int col = j >> 1;
#pragma unroll
        for (int ks = 0; ks < C::NK; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) rr[ks][e] = src[(16 * ks + 8 * kg + e) * (D / 2) + col];
    }
    build_bucket_table(table, boundaries, tid, C::THREADS);
    {
#pragma unroll
        for (int ks = 0; ks < C::NK; ++ks) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float r = rr[ks][e];
                if constexpr (kBf16 && NT == 3) {
                    const __bf16 t0 = bf16_trunc(r);
                    const float r1 = r - bf16_value(t0);
                    const __bf16 t1 = bf16_trunc(r1);
                    const __bf16 t2 = bf16_trunc(r1 - bf16_value(t1));
                    a_t[0][ks][e] = t0; a_t[1][ks][e] = t1; a_t[2][ks][e] = t2;
                } else if constexpr (kBf16) {
                    const __bf16 t0 = bf16_nearest(r);
                    a_t[0][ks][e] = t0; a_t[1][ks][e] = bf16_nearest(r - bf16_value(t0));
                } else {
                    const _Float16 hi = _Float16(r);
                    a_hi[ks][e] = hi;
                    a_lo[ks][e] = _Float16((r - float(hi)) * 4096.0f);
                }
            }
        }
    }
    const float inv_w = table.inv_w, offset = table.offset;
    const bool slow = table.slow != 0;
    const uint32_t copy8 = 8u * uint32_t(n32);

    auto stage = [&](int64_t tile, Origin org, int buf) {
        const int live = rows_in(tile);
        const int64_t row0 = tile * C::TT;
        float ss_mine = 0.0f, up_mine = 1.0f;
#pragma unroll
        for (int p = 0; p < C::PASSES; ++p) {
            const int r = p * C::ROWS_PER_PASS + row_in_pass;
            float e[8];
            const uint32_t w[4] = {pre[p].x, pre[p].y, pre[p].z, pre[p].w};
            float ss = 0.0f, mx = 0.0f;
            if constexpr (kBf16) {
                // sum of squares straight from the packed pairs (v_dot2_f32_bf16)
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const bf16x2 v = __builtin_bit_cast(bf16x2, w[i]);
                    ss = __builtin_amdgcn_fdot2_f32_bf16(v, v, ss, false);
                }
            } else {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    e[2 * i] = load_elem<DT>(uint16_t(w[i] & 0xffffu));
                    e[2 * i + 1] = load_elem<DT>(uint16_t(w[i] >> 16));
                }
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    ss = __builtin_fmaf(e[i], e[i], ss);
                    mx = __builtin_fmaxf(mx, __builtin_fabsf(e[i]));
                }
            }
            // all-reduce over the CPR lanes of the row, in the VALU (quad swaps, mirrors, row swap)
            ss += dpp_f32<0xB1>(ss);      // lane ^ 1
            ss += dpp_f32<0x4E>(ss);      // lane ^ 2
            ss += dpp_f32<0x141>(ss);     // mirror of 8: the other quad
            if (C::CPR >= 16) ss += dpp_f32<0x140>(ss);   // mirror of 16
            if (C::CPR >= 32) {
                const auto sw = __builtin_amdgcn_permlane16_swap(float_to_bits(ss), float_to_bits(ss), false, false);
                ss = bits_to_float(sw[0]) + bits_to_float(sw[1]);
            }
            float up = 1.0f;
            uint4v h = pre[p];
            if constexpr (!kBf16) {
                mx = __builtin_fmaxf(mx, dpp_f32<0xB1>(mx));
                mx = __builtin_fmaxf(mx, dpp_f32<0x4E>(mx));
                mx = __builtin_fmaxf(mx, dpp_f32<0x141>(mx));
                if (C::CPR >= 16) mx = __builtin_fmaxf(mx, dpp_f32<0x140>(mx));
                if (C::CPR >= 32) {
                    const auto mw = __builtin_amdgcn_permlane16_swap(float_to_bits(mx), float_to_bits(mx), false, false);
                    mx = __builtin_fmaxf(bits_to_float(mw[0]), bits_to_float(mw[1]));
                }
                int ex = int((float_to_bits(mx) >> 23) & 0xffu) - 127;
                if (ex < -126 || ex > 126) ex = 0;   // zero / subnormal / non-finite rows: no scaling
                const float down = bits_to_float(uint32_t(127 - ex) << 23);
                up = bits_to_float(uint32_t(127 + ex) << 23);
                h.x = pack_h2(_Float16(e[0] * down), _Float16(e[1] * down));
                h.y = pack_h2(_Float16(e[2] * down), _Float16(e[3] * down));
                h.z = pack_h2(_Float16(e[4] * down), _Float16(e[5] * down));
                h.w = pack_h2(_Float16(e[6] * down), _Float16(e[7] * down));
            }
            *reinterpret_cast<uint4v*>(&xs[buf][r * C::XS_STRIDE + chunk * 16]) = h;
            // every lane of a row holds the row's sum: the lane of chunk p keeps the one of pass p
            if (p == 0 || chunk == p) {
                ss_mine = ss;
                up_mine = up;
            }
        }
        // ---- norm, row factor and the norm's store: once per tile, by the lanes of chunks 0..PASSES-1,
        // each for the row it met in the pass of its chunk number ---------------------------------
        static_assert(C::CPR >= C::PASSES, "a row has a lane for every pass");
        // v_sqrt_f32 (1 ulp), with a sum of squares in the subnormal range scaled into the normal one
        const bool tiny = ss_mine < 0x1p-96f;
        const float nrm_s = __builtin_amdgcn_sqrtf(tiny ? ss_mine * 0x1p64f : ss_mine);
        const float nrm = tiny ? nrm_s * 0x1p-32f : nrm_s;
        if (chunk < C::PASSES) {
            const int r = chunk * C::ROWS_PER_PASS + row_in_pass;
            inv_s[buf][r] = up_mine * __builtin_amdgcn_rcpf(nrm + 1e-10f);
            if (r < live) {
                if (PAGED) {
                    int head, is_v;
                    uint8_t* dst = paged_row(org, r, head, is_v);
                    if (dst) *reinterpret_cast<float*>(dst + pd.H * (D / 2) + 4 * head) = nrm;
                } else if (pd.append_n == 0u) {      // uniform
                    (norms + row0)[r] = nrm;
                } else {
                    norms[appended_row(org, r)] = nrm;
                }
            }
        }
    };

    // packed rows of a tile: LDS -> global, 16 bytes per lane
    auto store_tile = [&](int64_t tile, Origin org, const uint8_t* ob) {
        constexpr int OC = D / 32;   // 16-byte chunks per packed row
        const int live = rows_in(tile);
        const int64_t row0 = tile * C::TT;
        for (int c = tid; c < C::TT * OC; c += C::THREADS) {
            const int r = c / OC, q = c % OC;
            if (r < live) {
                const uint2v lo = *reinterpret_cast<const uint2v*>(&ob[r * C::OUT_STRIDE + q * 16]);
                const uint2v hi = *reinterpret_cast<const uint2v*>(&ob[r * C::OUT_STRIDE + q * 16 + 8]);
                uint4v v = {lo.x, lo.y, hi.x, hi.y};
                if (PAGED) {
                    int head, is_v;
                    uint8_t* dst = paged_row(org, r, head, is_v);
                    if (dst) {
                        dst += head * (D / 2) + 16 * q;
                        if (pd.wide) {
                            *reinterpret_cast<uint4v*>(dst) = v;
                        } else {
                            uint32_t* d4 = reinterpret_cast<uint32_t*>(dst);
                            d4[0] = v.x; d4[1] = v.y; d4[2] = v.z; d4[3] = v.w;
                        }
                    }
                } else if (pd.append_n == 0u) {          // uniform: chunk c of the tile is chunk c of its rows
                    __builtin_nontemporal_store(v, reinterpret_cast<uint4v*>(packed + row0 * (D / 2)) + c);
                } else {
                    __builtin_nontemporal_store(v, reinterpret_cast<uint4v*>(packed + appended_row(org, r) * (D / 2)) + q);
                }
            }
        }
    };

    int64_t tile = blockIdx.x;

    // ---- software pipeline (head_dim 128) -------------------------------------------------------
    // The unit of work is a block of 32 rows.  The matrix instructions of block u + 1 are issued
    // between the lookups and compares that bucketize block u, so that a wavefront keeps both the
    // matrix pipe and the vector ALU busy instead of alternating between them (two wavefronts
    // share a SIMD; phases that alternate fall into step and leave one of the two units idle).
    // Per tile: [MFMA (tile, 1) | finish (tile, 0)], stage tile + 1, barrier,
    //           [MFMA (tile + 1, 0) | finish (tile, 1)], barrier, store tile.
    if constexpr (kPipe) {
        if (!slow && tile < num_tiles) {
            const int64_t G = gridDim.x;
            auto pipe = [&](int mbuf, int mtb, float16v& acc_out, int fbuf, int ftb,
                            const float16v& acc_in, uint8_t* ob) {
                const uint8_t* brow = &xs[mbuf][(32 * mtb + n32) * C::XS_STRIDE + kg * 16];
                const float inv = inv_s[fbuf][32 * ftb + n32];
                float16v acc;
                uint2v cell[16];
                float yv[16];
                uint32_t word[2] = {0u, 0u};
                // Step st looks up element ord(st) and compares the element of step st - 4.  The order
                // is that of the nibbles of the two output words from the top down (byte j = idx[2j] <<
                // 4 | idx[2j+1]), so that a word is built as word = (word << 4) + base + (thr < y):
                // two instructions per element for index and packing.
                auto ord = [](int st) { return 8 * (st >> 3) + (6 - 2 * ((st & 7) >> 1)) + (st & 1); };
                constexpr int kTerms = kBf16 ? NT : 2;           // fp16 rows: hi and lo, an accumulator each
                constexpr int kSteps = 8 * kTerms > 20 ? 8 * kTerms : 20;
                float16v acc_lo;
#pragma unroll
                for (int st = 0; st < kSteps; ++st) {
                    if (st < 8 * kTerms) {
                        const int ks = st / kTerms, t = kTerms - 1 - st % kTerms;
                        // (the first product starts from the constant 0, not from cleared registers)
                        if constexpr (kBf16) {
                            const bf16x8 b = *reinterpret_cast<const bf16x8*>(brow + ks * 32);
                            if (st == 0) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_t[t][ks], b, float16v{}, 0, 0, 0);
                            else acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_t[t][ks], b, acc, 0, 0, 0);
                        } else {
                            const half8 b = *reinterpret_cast<const half8*>(brow + ks * 32);
                            if (t == 1) acc_lo = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_lo[ks], b, ks == 0 ? float16v{} : acc_lo, 0, 0, 0);
                            else acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_hi[ks], b, ks == 0 ? float16v{} : acc, 0, 0, 0);
                        }
                    }
                    if (st < 16) {
                        yv[st] = acc_in[ord(st)] * inv;
                        cell[st] = bucket_cell(yv[st], inv_w, offset, copy8);
                    }
                    if (st >= 4 && st < 20) {
                        const int e = st - 4;
                        word[e >> 3] = (word[e >> 3] << 4) + cell[e].y + (bits_to_float(cell[e].x) < yv[e] ? 1u : 0u);
                    }
                }
                const uint2v o = {word[0], word[1]};
                *reinterpret_cast<uint2v*>(&ob[(32 * ftb + n32) * C::OUT_STRIDE + 16 * cb + 8 * kg]) = o;
                if constexpr (kBf16) {
                    acc_out = acc;
                } else {
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc_out[i] = __builtin_fmaf(acc_lo[i], kLoScale, acc[i]);
                }
            };

            Origin org = origin_of(blockIdx.x);
            stage(tile, org, 0);                   // its loads were issued at the top of the kernel
            if (tile + G < num_tiles) issue_loads(tile + G);
            __syncthreads();
            float16v acc_a = {}, acc_b = {};
            {   // block (tile, 0): nothing to overlap with yet
                const uint8_t* brow = &xs[0][n32 * C::XS_STRIDE + kg * 16];
                if constexpr (kBf16) {
#pragma unroll
                    for (int st = 0; st < 8 * NT; ++st) {
                        const int ks = st / NT, t = NT - 1 - st % NT;
                        const bf16x8 b = *reinterpret_cast<const bf16x8*>(brow + ks * 32);
                        acc_a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_t[t][ks], b, acc_a, 0, 0, 0);
                    }
                } else {
                    float16v lo = {};
#pragma unroll
                    for (int ks = 0; ks < C::NK; ++ks) {
                        const half8 b = *reinterpret_cast<const half8*>(brow + ks * 32);
                        acc_a = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_hi[ks], b, acc_a, 0, 0, 0);
                        lo = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_lo[ks], b, lo, 0, 0, 0);
                    }
#pragma unroll
                    for (int i = 0; i < 16; ++i) acc_a[i] = __builtin_fmaf(lo[i], kLoScale, acc_a[i]);
                }
            }
            for (int it = 0; tile < num_tiles; tile += G, ++it) {
                const int cur = it & 1;
                const int64_t next = tile + G;
                const bool has_next = next < num_tiles;
                uint8_t* ob = outs + cur * kOutBytes;
                pipe(cur, 1, acc_b, cur, 0, acc_a, ob);
                const Origin next_org = advance(org);
                if (has_next) {
                    stage(next, next_org, cur ^ 1);
                    if (next + G < num_tiles) issue_loads(next + G);
                }
                __syncthreads();                      // tile + 1 is staged
                // past the last tile the matrix instructions run on stale rows and their result is dropped
                pipe(cur ^ 1, 0, acc_a, cur, 1, acc_b, ob);
                __syncthreads();                      // the packed rows of this tile are complete
                store_tile(tile, org, ob);
                org = next_org;
            }
            return;
        }
    }

    Origin org = origin_of(blockIdx.x);
    if (tile < num_tiles) stage(tile, org, 0);     // its loads were issued at the top of the kernel
    __syncthreads();

    for (int it = 0; tile < num_tiles; tile += gridDim.x, ++it) {
        const int cur = it & 1;
        const int64_t next = tile + gridDim.x;
        if (next < num_tiles) issue_loads(next);

        // ---- rotate + bucketize + pack ---------------------------------------
        for (int tb = tb0; tb < C::TB; tb += C::TB_STEP) {
            float16v acc_hi = {}, acc_lo = {};
            const uint8_t* brow = &xs[cur][(32 * tb + n32) * C::XS_STRIDE + kg * 16];
            if constexpr (kBf16) {
                // the small terms first, so that they are not rounded away against the large one
#pragma unroll
                for (int t = NT - 1; t >= 0; --t)
#pragma unroll
                    for (int ks = 0; ks < C::NK; ++ks) {
                        const bf16x8 b = *reinterpret_cast<const bf16x8*>(brow + ks * 32);
                        acc_hi = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_t[t][ks], b, acc_hi, 0, 0, 0);
                    }
            } else {
#pragma unroll
                for (int ks = 0; ks < C::NK; ++ks) {
                    const half8 b = *reinterpret_cast<const half8*>(brow + ks * 32);
                    acc_hi = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_hi[ks], b, acc_hi, 0, 0, 0);
                    acc_lo = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_lo[ks], b, acc_lo, 0, 0, 0);
                }
            }
            const float inv = inv_s[cur][32 * tb + n32];
            float yv[16];
#pragma unroll
            for (int i = 0; i < 16; ++i)
                yv[i] = (kBf16 ? acc_hi[i] : __builtin_fmaf(acc_lo[i], kLoScale, acc_hi[i])) * inv;
            uint32_t idx[16];
            if (!slow) {
#pragma unroll
                for (int i = 0; i < 16; ++i) idx[i] = bucket_fast(yv[i], inv_w, offset, copy8);
            } else {
#pragma unroll
                for (int i = 0; i < 16; ++i) idx[i] = bucket_slow(table, yv[i]);
            }
            uint2v o;
            o.x = (idx[0] << 4 | idx[1]) | (idx[2] << 4 | idx[3]) << 8 | (idx[4] << 4 | idx[5]) << 16 |
                  (idx[6] << 4 | idx[7]) << 24;
            o.y = (idx[8] << 4 | idx[9]) | (idx[10] << 4 | idx[11]) << 8 | (idx[12] << 4 | idx[13]) << 16 |
                  (idx[14] << 4 | idx[15]) << 24;
            *reinterpret_cast<uint2v*>(&outs[(32 * tb + n32) * C::OUT_STRIDE + 16 * cb + 8 * kg]) = o;
        }
        __syncthreads();

        store_tile(tile, org, outs);
        org = advance(org);
        if (next < num_tiles) stage(next, org, cur ^ 1);
        __syncthreads();
    }
}

// bf16 terms of the matrix: three (exact) on request, and where the count does not matter (the
// fp16 route: one instantiation)
template <int D, int DT>
int bf16_terms() {
    if (DT != FQ_BF16) return 3;
    return fq_host::option(FQ_OPT_COMPRESS_THREE_TERMS) != 0 ? 3 : 2;
}

template <int D, int DT>
int launch_compress(const void* x, const float* re, const float* ro, const float* bnd, uint8_t* packed,
                    float* norms, int64_t M, int num_cus, hipStream_t s, const PagedDest& pd = PagedDest{}) {
    using C = CompressCfg<D>;
    const int64_t tiles = (M + C::TT - 1) / C::TT;
    const int64_t cap = int64_t(num_cus) * 2;
    const unsigned grid = unsigned(tiles < cap ? tiles : cap);
    if (bf16_terms<D, DT>() == 3)
        hipLaunchKernelGGL((tq4_compress_kernel<D, DT, false, 3>), dim3(grid), dim3(C::THREADS), 0, s,
                           reinterpret_cast<const uint4v*>(x), re, ro, bnd, packed, norms, M, tiles, pd);
    else
        hipLaunchKernelGGL((tq4_compress_kernel<D, DT, false, 2>), dim3(grid), dim3(C::THREADS), 0, s,
                           reinterpret_cast<const uint4v*>(x), re, ro, bnd, packed, norms, M, tiles, pd);
    return fq_host::check_launch();
}

template <int D, int DT>
int launch_compress_store(const void* key, const float* re, const float* ro, const float* bnd, const PagedDest& pd,
                          int num_cus, hipStream_t s) {
    using C = CompressCfg<D>;
    const int64_t M = 2 * pd.rows_k;
    const int64_t tiles = (M + C::TT - 1) / C::TT;
    const int64_t cap = int64_t(num_cus) * 2;
    const unsigned grid = unsigned(tiles < cap ? tiles : cap);
    if (bf16_terms<D, DT>() == 3)
        hipLaunchKernelGGL((tq4_compress_kernel<D, DT, true, 3>), dim3(grid), dim3(C::THREADS), 0, s,
                           reinterpret_cast<const uint4v*>(key), re, ro, bnd, static_cast<uint8_t*>(nullptr),
                           static_cast<float*>(nullptr), M, tiles, pd);
    else
        hipLaunchKernelGGL((tq4_compress_kernel<D, DT, true, 2>), dim3(grid), dim3(C::THREADS), 0, s,
                           reinterpret_cast<const uint4v*>(key), re, ro, bnd, static_cast<uint8_t*>(nullptr),
                           static_cast<float*>(nullptr), M, tiles, pd);
    return fq_host::check_launch();
}

}  // namespace fq

namespace fq_host {
int device_cu_count() {
    static thread_local int cached_dev = -1;
    static thread_local int cached_cus = 0;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (dev != cached_dev) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
            cus = 256;
        cached_dev = dev;
        cached_cus = cus;
    }
    return cached_cus;
}
}  // namespace fq_host

extern "C" int fq_tq4_compress(const void* x, int x_dtype, const float* rot_T_even,
                               const float* rot_T_odd, const float* boundaries, uint8_t* packed,
                               float* norms, int64_t M, int D, void* stream) {
    using namespace fq;
    if (M < 0) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (x_dtype != FQ_F16 && x_dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (M == 0) return FQ_OK;
    if (!x || !rot_T_even || !rot_T_odd || !boundaries || !packed || !norms) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(x, 16) || !fq_host::aligned(packed, 16) || !fq_host::aligned(norms, 4))
        return FQ_ERR_MISALIGNED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int cus = fq_host::device_cu_count();
#define FQ_COMPRESS_CASE(DD)                                                                              \
    case DD:                                                                                              \
        return x_dtype == FQ_F16                                                                          \
                   ? launch_compress<DD, FQ_F16>(x, rot_T_even, rot_T_odd, boundaries, packed, norms, M, cus, s) \
                   : launch_compress<DD, FQ_BF16>(x, rot_T_even, rot_T_odd, boundaries, packed, norms, M, cus, s);
    switch (D) {
        FQ_COMPRESS_CASE(64)
        FQ_COMPRESS_CASE(128)
        FQ_COMPRESS_CASE(256)
        default: return FQ_ERR_UNSUPPORTED_DIM;
    }
#undef FQ_COMPRESS_CASE
}

// Shares the compress kernel, and so its rotation precision: bf16 rows of head_dim 64 / 128 against two
// bf16 terms of the matrix unless FQ_OPT_COMPRESS_THREE_TERMS asks for the third (compress_matrix_terms).
extern "C" int fq_tq4_compress_append(const void* x, int x_dtype, const float* rot_T_even, const float* rot_T_odd,
                                      const float* boundaries, uint8_t* packed, float* norms, int64_t outer,
                                      int64_t n_new, int64_t capacity, int64_t position, int D, void* stream) {
    using namespace fq;
    if (outer < 0 || n_new < 0 || capacity < 0 || position < 0 || position + n_new > capacity) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (x_dtype != FQ_F16 && x_dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (outer == 0 || n_new == 0) return FQ_OK;
    if (outer * n_new > 0x7fffffffLL || n_new > 0x7fffffffLL) return FQ_ERR_BAD_SHAPE;   // 32-bit row arithmetic in the kernel
    if (!x || !rot_T_even || !rot_T_odd || !boundaries || !packed || !norms) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(x, 16) || !fq_host::aligned(packed, 16) || !fq_host::aligned(norms, 4))
        return FQ_ERR_MISALIGNED;
    PagedDest pd{};
    pd.append_n = uint32_t(n_new);
    pd.append_cap = capacity;
    pd.append_pos = position;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int cus = fq_host::device_cu_count();
    const int64_t M = outer * n_new;
#define FQ_APPEND_CASE(DD)                                                                                         \
    case DD:                                                                                                       \
        return x_dtype == FQ_F16                                                                                   \
                   ? launch_compress<DD, FQ_F16>(x, rot_T_even, rot_T_odd, boundaries, packed, norms, M, cus, s, pd)  \
                   : launch_compress<DD, FQ_BF16>(x, rot_T_even, rot_T_odd, boundaries, packed, norms, M, cus, s, pd);
    switch (D) {
        FQ_APPEND_CASE(64)
        FQ_APPEND_CASE(128)
        FQ_APPEND_CASE(256)
        default: return FQ_ERR_UNSUPPORTED_DIM;
    }
#undef FQ_APPEND_CASE
}

// Rotation precision as in fq_tq4_compress: two bf16 matrix terms by default for bf16 rows of head_dim
// 64 / 128, three with FQ_OPT_COMPRESS_THREE_TERMS (compress_matrix_terms).
extern "C" int fq_tq4_compress_store(const void* key, const void* value, int x_dtype,
                                     const float* rot_T_even, const float* rot_T_odd, const float* boundaries,
                                     uint8_t* kv_cache, const int64_t* slot_mapping,
                                     int64_t num_tokens, int64_t num_mapped, int H_KV, int D,
                                     int64_t num_slots, void* stream) {
    using namespace fq;
    if (num_tokens < 0 || num_mapped < 0 || num_mapped > num_tokens || H_KV <= 0 || num_slots < 0) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (x_dtype != FQ_F16 && x_dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (num_tokens == 0 || num_mapped == 0) return FQ_OK;
    if (!key || !value || !rot_T_even || !rot_T_odd || !boundaries || !kv_cache || !slot_mapping) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(key, 16) || !fq_host::aligned(value, 16) || !fq_host::aligned(kv_cache, 16) ||
        !fq_host::aligned(slot_mapping, 8))
        return FQ_ERR_MISALIGNED;
    // the kernel counts tokens in 32 bits and divides by the head count in float32
    if (num_tokens > 0x7fffffffLL || H_KV > 65536 || num_tokens * H_KV > (int64_t(1) << 40)) return FQ_ERR_BAD_SHAPE;
    PagedDest pd{};
    pd.x_value = static_cast<const uint4v*>(value);
    pd.cache = kv_cache;
    pd.slots = slot_mapping;
    pd.rows_k = num_tokens * H_KV;
    pd.tokens = uint32_t(num_tokens);
    pd.num_slots = num_slots;
    pd.mapped = int(num_mapped);
    pd.H = H_KV;
    pd.wide = ((int64_t(H_KV) * (D + 8)) % 16 == 0 && (int64_t(H_KV) * (D / 2 + 4)) % 16 == 0 && (D / 2) % 16 == 0) ? 1 : 0;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int cus = fq_host::device_cu_count();
#define FQ_STORE_CASE(DD)                                                                            \
    case DD:                                                                                         \
        return x_dtype == FQ_F16                                                                     \
                   ? launch_compress_store<DD, FQ_F16>(key, rot_T_even, rot_T_odd, boundaries, pd, cus, s)  \
                   : launch_compress_store<DD, FQ_BF16>(key, rot_T_even, rot_T_odd, boundaries, pd, cus, s);
    switch (D) {
        FQ_STORE_CASE(64)
        FQ_STORE_CASE(128)
        FQ_STORE_CASE(256)
        default: return FQ_ERR_UNSUPPORTED_DIM;
    }
#undef FQ_STORE_CASE
}
