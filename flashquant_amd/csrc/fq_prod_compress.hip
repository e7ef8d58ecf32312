// TurboQuantProd key compress for gfx950: 3-bit Lloyd-Max index + 1 sign bit of the
// sketched residual per coordinate, packed as one nibble (sign << 3 | index), plus the
// row norm and the residual norm.
//
// Operator: TurboQuantProd.quantize (src/flashquant/core/quantizer.py:285-304):
//   n = ||x||, y = (x / (n + 1e-10)) R^T, idx = #{boundaries < y}        (the bits-1 codebook)
//   resid = x - (centroids[idx] R) n,  gamma = ||resid||,  signs = sign(resid S^T), 0 -> +1
// The residual is handled in rotated space: resid R^T = (n + 1e-10) y - n centroids[idx]
// has the same norm (R is orthogonal) and resid S^T = (resid R^T) (S R^T)^T, so the second
// product uses the matrix W = S R^T, which the caller computes once.
//
// Both products run on the float32 MFMA (v_mfma_f32_16x16x4_f32): the signs of small
// projections are decided at float32 accuracy, as in the reference.  A workgroup of 4
// wavefronts takes 16 rows at a time; wavefront w owns output columns 16w..16w+15 and
// 64+16w.. of both products and keeps those columns of R and W in registers for the
// kernel's lifetime.
#include "fq_common.hpp"
#include "fq_device.hpp"

namespace fq {

constexpr int kPcRows = 16;
constexpr int kPcStride = 128 + 4;   // floats per staged row

template <int DT>
__global__ __launch_bounds__(256) void prod_compress_kernel(
    const uint4v* __restrict__ x, const float* __restrict__ R, int rot_col_major, const float* __restrict__ W,
    const float* __restrict__ boundaries, const float* __restrict__ centroids, uint32_t* __restrict__ packed,
    float* __restrict__ norms, float* __restrict__ gamma, int64_t M, int64_t num_tiles) {
    constexpr int D = 128;
    __shared__ float xs[kPcRows][kPcStride];   // normalised row, then the rotated residual
    __shared__ float ys[kPcRows][kPcStride];   // rotated row, then the projected residual
    __shared__ float bnd[8], cen[8];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n16 = lane & 15, g4 = lane >> 4;
    const int row = tid >> 4, c8 = tid & 15;   // elementwise phases: 8 coordinates of one row

    if (tid < 7) bnd[tid] = boundaries[tid];
    if (tid == 7) bnd[7] = __builtin_inff();
    if (tid >= 8 && tid < 16) cen[tid - 8] = centroids[tid - 8];

    float rb[2][4][8], wb[2][4][8];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        load_rotation_any<D>(R, rot_col_major != 0, true, 16 * (wave + 4 * i), n16, g4, rb[i]);
        load_rotation_any<D>(W, false, true, 16 * (wave + 4 * i), n16, g4, wb[i]);
    }
    __syncthreads();

    for (int64_t tile = blockIdx.x; tile < num_tiles; tile += gridDim.x) {
        const int64_t grow = tile * kPcRows + row;
        const bool live = grow < M;
        // ---- norm, normalised row --------------------------------------------------------
        float e[8];
        {
            const uint4v raw = live ? x[grow * (D / 8) + c8] : uint4v{0, 0, 0, 0};
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                e[2 * i] = load_elem<DT>(uint16_t(w[i] & 0xffffu));
                e[2 * i + 1] = load_elem<DT>(uint16_t(w[i] >> 16));
            }
        }
        float ss = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ss = __builtin_fmaf(e[i], e[i], ss);
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) ss += xor_shuffle(ss, m);
        const float nrm = __builtin_sqrtf(ss);
        const float den = nrm + 1e-10f;
#pragma unroll
        for (int i = 0; i < 8; ++i) xs[row][8 * c8 + i] = e[i] / den;
        __syncthreads();

        // ---- y = xhat R^T ------------------------------------------------------------------
        float a[4][8];
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int k = 0; k < 8; ++k) a[j][k] = xs[n16][32 * j + 8 * g4 + k];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float4v acc = rotate_block<D>(a, rb[i]);
#pragma unroll
            for (int r = 0; r < 4; ++r) ys[4 * g4 + r][16 * (wave + 4 * i) + n16] = acc[r];
        }
        __syncthreads();

        // ---- 3-bit index, rotated residual, its norm ---------------------------------------------
        uint32_t nib = 0;
        float g2 = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float y = ys[row][8 * c8 + i];
            uint32_t idx = 0;
#pragma unroll
            for (int b = 0; b < 7; ++b) idx += (bnd[b] < y) ? 1u : 0u;
            const float r = den * y - nrm * cen[idx];
            g2 = __builtin_fmaf(r, r, g2);
            xs[row][8 * c8 + i] = r;
            nib |= idx << (4 * i);
        }
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) g2 += xor_shuffle(g2, m);
        __syncthreads();

        // ---- projection of the residual: (resid R^T) W^T ---------------------------------------------
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int k = 0; k < 8; ++k) a[j][k] = xs[n16][32 * j + 8 * g4 + k];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const float4v acc = rotate_block<D>(a, wb[i]);
#pragma unroll
            for (int r = 0; r < 4; ++r) ys[4 * g4 + r][16 * (wave + 4 * i) + n16] = acc[r];
        }
        __syncthreads();

        // ---- sign bits, pack: byte j = nibble(2j) << 4 | nibble(2j + 1) ------------------------------------
        uint32_t word = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t neg = ys[row][8 * c8 + i] < 0.0f ? 8u : 0u;
            const uint32_t nb = ((nib >> (4 * i)) & 7u) | neg;
            word |= nb << (8 * (i >> 1) + ((i & 1) ? 0 : 4));
        }
        if (live) {
            packed[grow * (D / 8) + c8] = word;
            if (c8 == 0) {
                norms[grow] = nrm;
                gamma[grow] = __builtin_sqrtf(g2);
            }
        }
        // the next tile's first barrier orders its xs writes after this tile's reads of xs;
        // ys is rewritten only after that barrier as well
    }
}

}  // namespace fq

namespace fq_host {
int device_cu_count();
}

extern "C" int fq_prod_compress(const void* x, int x_dtype, const float* rotation, int rotation_col_major,
                                const float* sketch_rot, const float* boundaries, const float* centroids,
                                uint8_t* packed, float* norms, float* residual_norms, int64_t M, int D,
                                void* stream) {
    using namespace fq;
    if (M < 0) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D) || D != 128) return FQ_ERR_UNSUPPORTED_DIM;
    if (x_dtype != FQ_F16 && x_dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (M == 0) return FQ_OK;
    if (!x || !rotation || !sketch_rot || !boundaries || !centroids || !packed || !norms || !residual_norms)
        return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(x, 16) || !fq_host::aligned(packed, 4) || !fq_host::aligned(rotation, 16) ||
        !fq_host::aligned(sketch_rot, 16))
        return FQ_ERR_MISALIGNED;
    const int64_t tiles = (M + kPcRows - 1) / kPcRows;
    const int64_t cap = int64_t(fq_host::device_cu_count()) * 4;
    const unsigned grid = unsigned(tiles < cap ? tiles : cap);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint4v* xp = static_cast<const uint4v*>(x);
    uint32_t* pp = reinterpret_cast<uint32_t*>(packed);
    if (x_dtype == FQ_F16)
        hipLaunchKernelGGL(prod_compress_kernel<FQ_F16>, dim3(grid), dim3(256), 0, s, xp, rotation, rotation_col_major,
                           sketch_rot, boundaries, centroids, pp, norms, residual_norms, M, tiles);
    else
        hipLaunchKernelGGL(prod_compress_kernel<FQ_BF16>, dim3(grid), dim3(256), 0, s, xp, rotation, rotation_col_major,
                           sketch_rot, boundaries, centroids, pp, norms, residual_norms, M, tiles);
    return fq_host::check_launch();
}
