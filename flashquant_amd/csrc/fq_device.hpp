// Device helpers shared by the attention kernels: the byte -> (fp16, fp16) centroid
// table in LDS, cross-lane reductions that stay in the VALU, and the float32-MFMA
// head rotation.
#pragma once

#include "fq_common.hpp"

namespace fq {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kLutCopies = 64;                // one copy per lane: entry stride 256 bytes
constexpr int kLutWords = 256 * kLutCopies;   // per table (64 KB)
constexpr float kHalfMax = 65504.0f;
constexpr float kHalfSafe = 60000.0f;         // a P operand above this makes the softmax reference move
constexpr float kMaxLead = 16.0f;             // so does a score this many binary orders above the reference

__device__ __forceinline__ uint32_t byte_of(uint32_t w, int b) { return (w >> (8 * b)) & 0xffu; }

// Binary orders by which a value norm lies above 2^10 (0 for ordinary norms).  Added to a
// token's score when the softmax reference is chosen, it keeps weight * norm below 2^11, so the
// fp16 P operand of the second product cannot overflow whatever the norms are; numerator and
// denominator share the reference, so the result does not depend on it.
__device__ __forceinline__ float norm_bias(float vn) {
    const int ex = int((float_to_bits(vn) >> 23) & 0xffu) - 127;   // floor(log2 vn); Inf / NaN: 128
    return ex > 10 ? float(ex - 10) : 0.0f;
}

// Binary orders by which a row norm lies above 2^15 (0 for ordinary norms): a K or V tile holds
// fp16(centroid * norm / 2^excess), which always fits, and the power of two goes back in on the
// float32 side (the score, or the weight together with a raised softmax reference).
__device__ __forceinline__ int norm_excess(float n) {
    const int ex = int((float_to_bits(n) >> 23) & 0xffu) - 127;
    return ex > 14 ? ex - 14 : 0;
}

// LDS byte address of table entry `byte K of w` in the copy of this lane: the entry
// stride is 256 bytes and lane_off = 4 * lane < 256, so the address is the two bytes
// (byte K of w, lane_off) side by side: one v_perm_b32 instead of extract, shift and add.
template <int K>
__device__ __forceinline__ uint32_t lut_addr(uint32_t w, uint32_t lane_off) {
    return __builtin_amdgcn_perm(w, lane_off, 0x0C0C0000u | ((4u + K) << 8));
}
__device__ __forceinline__ uint32_t lds_word(const uint8_t* table, uint32_t addr) {
    return *reinterpret_cast<const uint32_t*>(table + addr);
}
// the four fp16 pairs of the four bytes of w
__device__ __forceinline__ uint4v lookup_word(const uint8_t* table, uint32_t w, uint32_t lane_off) {
    uint4v r;
    r.x = lds_word(table, lut_addr<0>(w, lane_off));
    r.y = lds_word(table, lut_addr<1>(w, lane_off));
    r.z = lds_word(table, lut_addr<2>(w, lane_off));
    r.w = lds_word(table, lut_addr<3>(w, lane_off));
    return r;
}
// byte BI of each of four words
template <int BI>
__device__ __forceinline__ uint4v lookup_column(const uint8_t* table, const uint32_t (&src)[4], uint32_t lane_off) {
    uint4v r;
    r.x = lds_word(table, lut_addr<BI>(src[0], lane_off));
    r.y = lds_word(table, lut_addr<BI>(src[1], lane_off));
    r.z = lds_word(table, lut_addr<BI>(src[2], lane_off));
    r.w = lds_word(table, lut_addr<BI>(src[3], lane_off));
    return r;
}

// Fills a 64-copy byte table: entry (byte, copy) = fp16 pair (centroid[byte >> 4],
// centroid[byte & 15]).  The 16 centroids are fetched once (lane l holds centroid
// l % 16); a wavefront then writes one byte's 64 copies per step, picking the two
// values with v_readlane, so the build is a short LDS-write loop with no memory
// latency inside it.
__device__ __forceinline__ void fill_byte_table(uint32_t* table, float mine, int wave, int waves, int lane) {
    for (int byte = wave; byte < 256; byte += waves) {
        const float hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), byte >> 4));
        const float lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), byte & 15));
        table[byte * kLutCopies + lane] = pack_h2(_Float16(hi), _Float16(lo));
    }
}
// Two tables in one 64 KB array of 256-byte rows: the K table in the lower 128 bytes of
// every row (lanes 0..31 write it, 32 copies, one per LDS bank of a half-wave) and the V
// table in the upper 128 bytes.  A K nibble is looked up as `nibble & k_mask` (15 for TQ4,
// 7 when bit 3 of the nibble is a sign bit), a V nibble as it is.  Lane l holds
// k_centroids[l & k_mask] and v_centroids[l & 15].
template <int WAVES>
__device__ __forceinline__ void fill_pair_tables(uint32_t* table, float mine_k, float mine_v, int k_mask, int wave,
                                                 int lane) {
    static_assert(WAVES == 8, "byte = wave + 8 i: the high nibble is i / 2, the low nibble wave or wave + 8");
    // the fp16 centroid of this lane; entries are then assembled on the scalar unit
    const int hk = int(__builtin_bit_cast(uint16_t, _Float16(mine_k)));
    const int hv = int(__builtin_bit_cast(uint16_t, _Float16(mine_v)));
    uint32_t* mine = table + lane;
    // low halves of this wavefront's entries (two possible low nibbles), shifted into place once
    const uint32_t klo[2] = {uint32_t(__builtin_amdgcn_readlane(hk, wave & k_mask)) << 16,
                             uint32_t(__builtin_amdgcn_readlane(hk, (wave + 8) & k_mask)) << 16};
    const uint32_t vlo[2] = {uint32_t(__builtin_amdgcn_readlane(hv, wave)) << 16,
                             uint32_t(__builtin_amdgcn_readlane(hv, wave + 8)) << 16};
#pragma unroll
    for (int hi = 0; hi < 16; ++hi) {
        // the high nibble is a compile-time lane index: one readlane per table and nibble
        const uint32_t kh = uint32_t(__builtin_amdgcn_readlane(hk, hi & k_mask));
        const uint32_t vh = uint32_t(__builtin_amdgcn_readlane(hv, hi));
#pragma unroll
        for (int lo = 0; lo < 2; ++lo) {
            const int i = 2 * hi + lo;                      // byte = wave + 8 i = 16 hi + (wave + 8 lo)
            const uint32_t ke = kh | klo[lo], ve = vh | vlo[lo];
            mine[wave * 64 + WAVES * 64 * i] = lane < 32 ? ke : ve;
        }
    }
}
__device__ __forceinline__ void build_byte_table(uint32_t* table, const float* __restrict__ centroids, int wave,
                                                 int waves, int lane) {
    fill_byte_table(table, centroids[lane & 15], wave, waves, lane);
}

// Cross-lane helpers that stay in the VALU (no LDS round trip).
template <int CTRL>
__device__ __forceinline__ float dpp_mov(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, false));
}
// max over lanes l and l ^ 16 (rows of 16 lanes swapped pairwise)
__device__ __forceinline__ float max_xor16(float v) {
    const uint32_t u = float_to_bits(v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return __builtin_fmaxf(bits_to_float(r[0]), bits_to_float(r[1]));
}
// max over lanes l and l ^ 32
__device__ __forceinline__ float max_xor32(float v) {
    const uint32_t u = float_to_bits(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return __builtin_fmaxf(bits_to_float(r[0]), bits_to_float(r[1]));
}
// sum over lanes l and l ^ 16, l and l ^ 32: one cross-lane vector instruction each, no LDS round trip
__device__ __forceinline__ float sum_xor16(float v) {
    const uint32_t u = float_to_bits(v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    return bits_to_float(r[0]) + bits_to_float(r[1]);
}
__device__ __forceinline__ float sum_xor32(float v) {
    const uint32_t u = float_to_bits(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    return bits_to_float(r[0]) + bits_to_float(r[1]);
}
// max over all lanes that share lane % GP
template <int GP>
__device__ __forceinline__ float max_same_head(float v) {
    if (GP <= 4) v = __builtin_fmaxf(v, dpp_mov<0x124>(v));   // row_ror:4
    if (GP <= 8) v = __builtin_fmaxf(v, dpp_mov<0x128>(v));   // row_ror:8
    return max_xor32(max_xor16(v));
}

// ---------------------------------------------------------------------------------------
// Head rotations: rows of D elements times the D x D rotation, float32 throughout, on the
// float32 MFMA (v_mfma_f32_16x16x4_f32), so that no splitting of the matrix is needed and
// the result matches a float32 matmul to rounding.  A workgroup (4 wavefronts) owns 16
// rows; wavefront w produces the 16-column blocks w, w + 4, ...
//
// The contraction index is permuted so that operands load as contiguous runs: MFMA step
// (j, e) with lane group g uses k = 32 j + 8 g + e, hence lane (m, g) holds the 8-element
// runs k = 32 j + 8 g .. + 7 of row m (A side) and of the matrix (B side).
// ---------------------------------------------------------------------------------------

constexpr int kRotRows = 16;

// B operand values of one 16-column block.  TRANSPOSED: out = x @ R.T (B[k][n] = R[col+n][k],
// contiguous in k); otherwise out = x @ R (B[k][n] = R[k][col+n], 16 lanes contiguous in n).
template <int D, bool TRANSPOSED>
__device__ __forceinline__ void load_rotation_block(const float* __restrict__ R, int col, int n, int g,
                                                    float (&b)[D / 32][8]) {
#pragma unroll
    for (int j = 0; j < D / 32; ++j) {
        if (TRANSPOSED) {
            const float4v* src = reinterpret_cast<const float4v*>(R + int64_t(col + n) * D + 32 * j + 8 * g);
            const float4v lo = src[0], hi = src[1];
            b[j][0] = lo.x; b[j][1] = lo.y; b[j][2] = lo.z; b[j][3] = lo.w;
            b[j][4] = hi.x; b[j][5] = hi.y; b[j][6] = hi.z; b[j][7] = hi.w;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) b[j][e] = R[int64_t(32 * j + 8 * g + e) * D + col + n];
        }
    }
}

// Rotation matrix given either row-major (element (i, j) at i*D + j) or column-major
// (at i + j*D, i.e. the transpose is the contiguous one, which is what a QR factor
// moved to the GPU looks like).  `x_times_Rt` selects out = x @ R.T, else out = x @ R.
template <int D>
__device__ __forceinline__ void load_rotation_any(const float* __restrict__ R, bool col_major, bool x_times_Rt,
                                                  int col, int n, int g, float (&b)[D / 32][8]) {
    // x @ R.T on a column-major R reads the same addresses as x @ R on a row-major one
    if (x_times_Rt != col_major) load_rotation_block<D, true>(R, col, n, g, b);
    else load_rotation_block<D, false>(R, col, n, g, b);
}

template <int D>
__device__ __forceinline__ float4v rotate_block(const float (&a)[D / 32][8], const float (&b)[D / 32][8]) {
    // four independent partial sums: a single accumulator would chain D/4 dependent MFMAs
    float4v acc[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < D / 32; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e)
            acc[e & 3] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[j][e], b[j][e], acc[e & 3], 0, 0, 0);
    return (acc[0] + acc[1]) + (acc[2] + acc[3]);
}

// ---------------------------------------------------------------------------------------
// The same rotations on the fp16 MFMA (v_mfma_f32_16x16x32_f16), 8 times the rate of the
// float32 one.  The matrix block is split once into two fp16 terms, b = hi + lo / 4096
// (22 significant bits); a row operand that is exact in fp16 after scaling by a power of
// two (fp16 / bf16 data) needs no split, so a block costs 2 MFMAs per 32 contraction
// indices and the products are exact.  Operand layout as rotate_block: lane (m, g) holds
// k = 32 j + 8 g + e.
// ---------------------------------------------------------------------------------------
template <int D>
__device__ __forceinline__ void split_rotation_block(const float (&b)[D / 32][8], half8 (&hi)[D / 32],
                                                     half8 (&lo)[D / 32]) {
#pragma unroll
    for (int j = 0; j < D / 32; ++j)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            // any rounding of the high term will do: the low term takes up the remainder
            const auto h2 = __builtin_amdgcn_cvt_pkrtz(b[j][e], b[j][e + 1]);
            const auto l2 = __builtin_amdgcn_cvt_pkrtz((b[j][e] - float(h2[0])) * 4096.0f, (b[j][e + 1] - float(h2[1])) * 4096.0f);
            hi[j][e] = h2[0]; hi[j][e + 1] = h2[1];
            lo[j][e] = l2[0]; lo[j][e + 1] = l2[1];
        }
}

template <int D>
__device__ __forceinline__ float4v rotate_block_f16(const half8 (&a)[D / 32], const half8 (&bhi)[D / 32],
                                                    const half8 (&blo)[D / 32]) {
    float4v acc_hi = {0.f, 0.f, 0.f, 0.f}, acc_lo = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < D / 32; ++j) {
        acc_hi = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], bhi[j], acc_hi, 0, 0, 0);
        acc_lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[j], blo[j], acc_lo, 0, 0, 0);
    }
    return acc_hi + acc_lo * (1.0f / 4096.0f);
}

// The same for rows that are bfloat16: they go to the bf16 MFMA as they are, against the matrix
// block split into three bf16 terms (3 x 8 bits: the float32 value exactly; bf16 keeps the float32
// exponent range, so the terms need no scaling and share one accumulator).
typedef __bf16 bf16v8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ __bf16 bf16_top(float f) {          // truncation: the next term takes up the rest
    return __builtin_bit_cast(__bf16, uint16_t(float_to_bits(f) >> 16));
}
__device__ __forceinline__ float bf16_as_float(__bf16 h) {
    return bits_to_float(uint32_t(__builtin_bit_cast(uint16_t, h)) << 16);
}
template <int D>
__device__ __forceinline__ void split_rotation_block_bf16(const float (&b)[D / 32][8], bf16v8 (&t)[3][D / 32]) {
#pragma unroll
    for (int j = 0; j < D / 32; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const __bf16 t0 = bf16_top(b[j][e]);
            const float r1 = b[j][e] - bf16_as_float(t0);
            const __bf16 t1 = bf16_top(r1);
            t[0][j][e] = t0;
            t[1][j][e] = t1;
            t[2][j][e] = bf16_top(r1 - bf16_as_float(t1));
        }
}
// The same three terms with the element pairs packed by v_perm_b32 and the remainders taken with an
// and + a subtraction (5.5 vector instructions per element instead of about 10).
template <int D>
__device__ __forceinline__ void split_rotation_block_bf16_packed(const float (&b)[D / 32][8], bf16v8 (&t)[3][D / 32]) {
#pragma unroll
    for (int j = 0; j < D / 32; ++j) {
        uint32_t w[3][4];
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            const uint32_t a0 = float_to_bits(b[j][e]), a1 = float_to_bits(b[j][e + 1]);
            w[0][e / 2] = __builtin_amdgcn_perm(a1, a0, 0x07060302u);            // top halves of the pair
            const float r0 = b[j][e] - bits_to_float(a0 & 0xffff0000u), r1 = b[j][e + 1] - bits_to_float(a1 & 0xffff0000u);
            const uint32_t c0 = float_to_bits(r0), c1 = float_to_bits(r1);
            w[1][e / 2] = __builtin_amdgcn_perm(c1, c0, 0x07060302u);
            const float s0 = r0 - bits_to_float(c0 & 0xffff0000u), s1 = r1 - bits_to_float(c1 & 0xffff0000u);
            w[2][e / 2] = __builtin_amdgcn_perm(float_to_bits(s1), float_to_bits(s0), 0x07060302u);
        }
#pragma unroll
        for (int k = 0; k < 3; ++k) t[k][j] = __builtin_bit_cast(bf16v8, uint4v{w[k][0], w[k][1], w[k][2], w[k][3]});
    }
}
template <int D>
__device__ __forceinline__ float4v rotate_block_bf16(const bf16v8 (&a)[D / 32], const bf16v8 (&t)[3][D / 32]) {
    float4v acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 2; k >= 0; --k)       // the small terms first
#pragma unroll
        for (int j = 0; j < D / 32; ++j) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], t[k][j], acc, 0, 0, 0);
    return acc;
}

// Wavefront-wide maximum (all 64 lanes receive it), in the VALU: rotations inside the rows
// of 16 lanes, then the row swaps.
__device__ __forceinline__ float wave_max(float v) {
    v = __builtin_fmaxf(v, dpp_mov<0x121>(v));   // row_ror:1
    v = __builtin_fmaxf(v, dpp_mov<0x122>(v));   // row_ror:2
    v = __builtin_fmaxf(v, dpp_mov<0x124>(v));   // row_ror:4
    v = __builtin_fmaxf(v, dpp_mov<0x128>(v));   // row_ror:8
    return max_xor32(max_xor16(v));
}

// 16-bit rows (fp16 / bf16 raw words, lane (m, g) holding k = 32 j + 8 g + e) as the fp16 A
// operand, scaled by one power of two for the whole 16-row block so that the largest
// element lies in [1, 2); `up` undoes the scaling on the result.
template <int D, int DT>
__device__ __forceinline__ void rows_as_f16(const uint4v (&raw)[D / 32], half8 (&a)[D / 32], float& up) {
    float v[D / 32][8];
    float mx = 0.0f;
#pragma unroll
    for (int j = 0; j < D / 32; ++j) {
        const uint32_t w[4] = {raw[j].x, raw[j].y, raw[j].z, raw[j].w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[j][2 * i] = load_elem<DT>(uint16_t(w[i] & 0xffffu));
            v[j][2 * i + 1] = load_elem<DT>(uint16_t(w[i] >> 16));
            mx = __builtin_fmaxf(mx, __builtin_fmaxf(__builtin_fabsf(v[j][2 * i]), __builtin_fabsf(v[j][2 * i + 1])));
        }
    }
    mx = wave_max(mx);
    int ex = int((float_to_bits(mx) >> 23) & 0xffu) - 127;
    if (ex < -100 || ex > 100) ex = 0;
    const float down = bits_to_float(uint32_t(127 - ex) << 23);
    up = bits_to_float(uint32_t(127 + ex) << 23);
#pragma unroll
    for (int j = 0; j < D / 32; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) a[j][e] = _Float16(v[j][e] * down);
}

// float32 rows (lane (m, g) holding k = 32 j + 8 g + e) as two fp16 terms, v = (hi + lo / 4096) * up,
// scaled by one power of two per 16-row block; with a split matrix block the product is
// hi.hi + (hi.lo + lo.hi) / 4096, accurate to about 2^-22 of the block's largest element.
template <int D>
__device__ __forceinline__ void rows_split_f16(const float (&v)[D / 32][8], half8 (&hi)[D / 32], half8 (&lo)[D / 32],
                                               float& up) {
    float mx = 0.0f;
#pragma unroll
    for (int j = 0; j < D / 32; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) mx = __builtin_fmaxf(mx, __builtin_fabsf(v[j][e]));
    mx = wave_max(mx);
    int ex = int((float_to_bits(mx) >> 23) & 0xffu) - 127;
    if (ex < -100 || ex > 100) ex = 0;
    const float down = bits_to_float(uint32_t(127 - ex) << 23);
    up = bits_to_float(uint32_t(127 + ex) << 23);
#pragma unroll
    for (int j = 0; j < D / 32; ++j)
#pragma unroll
        for (int e = 0; e < 8; e += 2) {
            const float a0 = v[j][e] * down, a1 = v[j][e + 1] * down;
            const auto h2 = __builtin_amdgcn_cvt_pkrtz(a0, a1);
            const auto l2 = __builtin_amdgcn_cvt_pkrtz((a0 - float(h2[0])) * 4096.0f, (a1 - float(h2[1])) * 4096.0f);
            hi[j][e] = h2[0]; hi[j][e + 1] = h2[1];
            lo[j][e] = l2[0]; lo[j][e + 1] = l2[1];
        }
}

template <int D>
__device__ __forceinline__ float4v rotate_block_f16x3(const half8 (&ahi)[D / 32], const half8 (&alo)[D / 32],
                                                      const half8 (&bhi)[D / 32], const half8 (&blo)[D / 32]) {
    float4v acc_hi = {0.f, 0.f, 0.f, 0.f}, acc_lo = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < D / 32; ++j) {
        acc_hi = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi[j], bhi[j], acc_hi, 0, 0, 0);
        acc_lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(ahi[j], blo[j], acc_lo, 0, 0, 0);
        acc_lo = __builtin_amdgcn_mfma_f32_16x16x32_f16(alo[j], bhi[j], acc_lo, 0, 0, 0);
    }
    return acc_hi + acc_lo * (1.0f / 4096.0f);
}

}  // namespace fq
