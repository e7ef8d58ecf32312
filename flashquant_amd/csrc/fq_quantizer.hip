// TurboQuantMSE / TurboQuantProd row operators for gfx950, any bit width up to 4:
//   quantize    n = ||x||, y = (x / (n + 1e-10)) R^T, idx = #{boundaries < y}
//   dequantize  out = (centroids[idx] R) n
//   residual    out = x - (centroids[idx] R) n, gamma = ||out||
//   project     out = x M^T, or its sign with 0 -> +1
// (TurboQuantMSE.quantize / dequantize, src/flashquant/core/quantizer.py:125-195, and the
// residual / sketch steps of TurboQuantProd.quantize and estimate_inner_product,
// quantizer.py:285-370).  These are the general operators behind the quantizer classes, in
// float32 throughout like the reference: the product runs on the float32 MFMA
// (v_mfma_f32_16x16x4_f32) so that bucket decisions and signs are taken at float32
// accuracy.  The serving path uses the specialised 4-bit kernels instead.
//
// A workgroup of 4 wavefronts takes 16 rows at a time: the rows are staged in LDS as
// float32, wavefront w computes output columns 16 (w + 4 i) .. + 15, the result goes back
// through LDS, and every thread finishes D / 16 consecutive coordinates of one row.
#include "fq_common.hpp"
#include "fq_device.hpp"

namespace fq {

enum QuantMode { QM_QUANTIZE = 0, QM_DEQUANTIZE = 1, QM_RESIDUAL = 2, QM_PROJECT = 3, QM_PROJECT_SIGN = 4 };

struct QuantArgs {
    const void* x;             // (M, D) rows: quantize, residual, project
    const int64_t* idx_in;     // (M, D): dequantize, residual
    const float* norms_in;     // (M,): dequantize, residual
    const float* mat;          // (D, D)
    int col_major;             // mat is stored transposed
    const float* table;        // boundaries (quantize) or centroids (dequantize, residual)
    int n_table;
    int64_t* idx_out;          // quantize
    float* f_out;              // dequantize, residual, project
    float* norms_out;          // quantize: norms; residual: residual norms
    int64_t M, tiles;
};

template <int XDT>
__device__ __forceinline__ float load_row_elem(const void* base, int64_t i) {
    if constexpr (XDT == FQ_F32) {
        return static_cast<const float*>(base)[i];
    } else {
        return load_elem<XDT>(static_cast<const uint16_t*>(base)[i]);
    }
}

template <int D, int MODE, int XDT>
__global__ __launch_bounds__(256) void quantizer_rows_kernel(const QuantArgs a) {
    constexpr int STRIDE = D + 4;
    constexpr int EPT = D / 16;        // coordinates per thread
    __shared__ float xs[16][STRIDE];
    __shared__ float ys[16][STRIDE];
    __shared__ float tab[16];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int n16 = lane & 15, g4 = lane >> 4;
    const int row = tid >> 4, c0 = (tid & 15) * EPT;

    if (tid < 16) tab[tid] = tid < a.n_table ? a.table[tid] : __builtin_inff();
    __syncthreads();
    // quantize, project: out = x M^T; dequantize, residual: out = c[idx] M
    constexpr bool kTimesMt = MODE == QM_QUANTIZE || MODE == QM_PROJECT || MODE == QM_PROJECT_SIGN;

    for (int64_t tile = blockIdx.x; tile < a.tiles; tile += gridDim.x) {
        const int64_t grow = tile * 16 + row;
        const bool live = grow < a.M;
        float e[EPT];
        float nrm = 0.0f;
        // ---- stage the left operand --------------------------------------------------------
        if (MODE == QM_DEQUANTIZE || MODE == QM_RESIDUAL) {
#pragma unroll
            for (int i = 0; i < EPT; ++i) {
                int64_t id = live ? a.idx_in[grow * D + c0 + i] : 0;
                id = id < 0 ? 0 : (id >= a.n_table ? a.n_table - 1 : id);
                xs[row][c0 + i] = tab[int(id)];
            }
            nrm = live ? a.norms_in[grow] : 0.0f;
        }
        if (MODE != QM_DEQUANTIZE) {
#pragma unroll
            for (int i = 0; i < EPT; ++i) e[i] = live ? load_row_elem<XDT>(a.x, grow * D + c0 + i) : 0.0f;
        }
        if (MODE == QM_QUANTIZE) {
            float ss = 0.0f;
#pragma unroll
            for (int i = 0; i < EPT; ++i) ss = __builtin_fmaf(e[i], e[i], ss);
#pragma unroll
            for (int m = 1; m < 16; m <<= 1) ss += xor_shuffle(ss, m);
            nrm = __builtin_sqrtf(ss);
            const float den = nrm + 1e-10f;
#pragma unroll
            for (int i = 0; i < EPT; ++i) xs[row][c0 + i] = e[i] / den;
        }
        if (MODE == QM_PROJECT || MODE == QM_PROJECT_SIGN) {
#pragma unroll
            for (int i = 0; i < EPT; ++i) xs[row][c0 + i] = e[i];
        }
        __syncthreads();

        // ---- product on the float32 MFMA ------------------------------------------------------
        float av[D / 32][8];
#pragma unroll
        for (int j = 0; j < D / 32; ++j)
#pragma unroll
            for (int k = 0; k < 8; ++k) av[j][k] = xs[n16][32 * j + 8 * g4 + k];
#pragma unroll
        for (int i = 0; i < D / 64; ++i) {
            float bv[D / 32][8];
            load_rotation_any<D>(a.mat, a.col_major != 0, kTimesMt, 16 * (wave + 4 * i), n16, g4, bv);
            const float4v acc = rotate_block<D>(av, bv);
#pragma unroll
            for (int r = 0; r < 4; ++r) ys[4 * g4 + r][16 * (wave + 4 * i) + n16] = acc[r];
        }
        __syncthreads();

        // ---- finish ----------------------------------------------------------------------------
        if (MODE == QM_QUANTIZE) {
#pragma unroll
            for (int i = 0; i < EPT; ++i) {
                const float y = ys[row][c0 + i];
                int id = 0;
#pragma unroll
                for (int b = 0; b < 15; ++b) id += (tab[b] < y) ? 1 : 0;     // unused slots hold +inf
                if (live) a.idx_out[grow * D + c0 + i] = id;
            }
            if (live && (tid & 15) == 0) a.norms_out[grow] = nrm;
        } else if (MODE == QM_DEQUANTIZE) {
#pragma unroll
            for (int i = 0; i < EPT; ++i)
                if (live) a.f_out[grow * D + c0 + i] = ys[row][c0 + i] * nrm;
        } else if (MODE == QM_RESIDUAL) {
            float g2 = 0.0f;
#pragma unroll
            for (int i = 0; i < EPT; ++i) {
                const float r = e[i] - ys[row][c0 + i] * nrm;
                g2 = __builtin_fmaf(r, r, g2);
                if (live) a.f_out[grow * D + c0 + i] = r;
            }
#pragma unroll
            for (int m = 1; m < 16; m <<= 1) g2 += xor_shuffle(g2, m);
            if (live && (tid & 15) == 0) a.norms_out[grow] = __builtin_sqrtf(g2);
        } else {
#pragma unroll
            for (int i = 0; i < EPT; ++i) {
                const float y = ys[row][c0 + i];
                const float v = MODE == QM_PROJECT ? y : (y < 0.0f ? -1.0f : 1.0f);
                if (live) a.f_out[grow * D + c0 + i] = v;
            }
        }
        // the staging of the next tile writes xs, which every wavefront has finished reading
        // before the barrier above; ys is rewritten only after the next tile's first barrier
    }
}

template <int D, int MODE>
int launch_rows_dtype(const QuantArgs& a, int x_dtype, unsigned grid, hipStream_t s) {
    if (MODE == QM_DEQUANTIZE || x_dtype == FQ_F32)
        hipLaunchKernelGGL((quantizer_rows_kernel<D, MODE, FQ_F32>), dim3(grid), dim3(256), 0, s, a);
    else if (x_dtype == FQ_F16)
        hipLaunchKernelGGL((quantizer_rows_kernel<D, MODE, FQ_F16>), dim3(grid), dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((quantizer_rows_kernel<D, MODE, FQ_BF16>), dim3(grid), dim3(256), 0, s, a);
    return fq_host::check_launch();
}

}  // namespace fq

namespace fq_host {
int device_cu_count();
}

namespace {

template <int MODE>
int launch_rows(fq::QuantArgs a, int x_dtype, int D, void* stream) {
    a.tiles = (a.M + 15) / 16;
    const int64_t cap = int64_t(fq_host::device_cu_count()) * 8;
    const unsigned grid = unsigned(a.tiles < cap ? a.tiles : cap);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (D) {
        case 64: return fq::launch_rows_dtype<64, MODE>(a, x_dtype, grid, s);
        case 128: return fq::launch_rows_dtype<128, MODE>(a, x_dtype, grid, s);
        default: return fq::launch_rows_dtype<256, MODE>(a, x_dtype, grid, s);
    }
}

bool row_dtype_ok(int dt) { return dt == FQ_F16 || dt == FQ_BF16 || dt == FQ_F32; }

}  // namespace

extern "C" int fq_mse_quantize(const void* x, int x_dtype, const float* rotation, int rotation_col_major,
                               const float* boundaries, int num_boundaries, int64_t* indices, float* norms,
                               int64_t M, int D, void* stream) {
    if (M < 0 || num_boundaries < 1 || num_boundaries > 15) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (!row_dtype_ok(x_dtype)) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (M == 0) return FQ_OK;
    if (!x || !rotation || !boundaries || !indices || !norms) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(rotation, 16) || !fq_host::aligned(indices, 8)) return FQ_ERR_MISALIGNED;
    fq::QuantArgs a{};
    a.x = x; a.mat = rotation; a.col_major = rotation_col_major; a.table = boundaries; a.n_table = num_boundaries;
    a.idx_out = indices; a.norms_out = norms; a.M = M;
    return launch_rows<fq::QM_QUANTIZE>(a, x_dtype, D, stream);
}

extern "C" int fq_mse_dequantize(const int64_t* indices, const float* norms, const float* rotation,
                                 int rotation_col_major, const float* centroids, int num_centroids, float* out,
                                 int64_t M, int D, void* stream) {
    if (M < 0 || num_centroids < 2 || num_centroids > 16) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (M == 0) return FQ_OK;
    if (!indices || !norms || !rotation || !centroids || !out) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(rotation, 16) || !fq_host::aligned(indices, 8)) return FQ_ERR_MISALIGNED;
    fq::QuantArgs a{};
    a.idx_in = indices; a.norms_in = norms; a.mat = rotation; a.col_major = rotation_col_major;
    a.table = centroids; a.n_table = num_centroids; a.f_out = out; a.M = M;
    return launch_rows<fq::QM_DEQUANTIZE>(a, FQ_F32, D, stream);
}

extern "C" int fq_mse_residual(const void* x, int x_dtype, const int64_t* indices, const float* norms,
                               const float* rotation, int rotation_col_major, const float* centroids,
                               int num_centroids, float* residual, float* residual_norms, int64_t M, int D,
                               void* stream) {
    if (M < 0 || num_centroids < 2 || num_centroids > 16) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (!row_dtype_ok(x_dtype)) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (M == 0) return FQ_OK;
    if (!x || !indices || !norms || !rotation || !centroids || !residual || !residual_norms) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(rotation, 16) || !fq_host::aligned(indices, 8)) return FQ_ERR_MISALIGNED;
    fq::QuantArgs a{};
    a.x = x; a.idx_in = indices; a.norms_in = norms; a.mat = rotation; a.col_major = rotation_col_major;
    a.table = centroids; a.n_table = num_centroids; a.f_out = residual; a.norms_out = residual_norms; a.M = M;
    return launch_rows<fq::QM_RESIDUAL>(a, x_dtype, D, stream);
}

extern "C" int fq_project_rows(const void* x, int x_dtype, const float* matrix, int matrix_col_major, int signs_only,
                               float* out, int64_t M, int D, void* stream) {
    if (M < 0) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (!row_dtype_ok(x_dtype)) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (M == 0) return FQ_OK;
    if (!x || !matrix || !out) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(matrix, 16)) return FQ_ERR_MISALIGNED;
    fq::QuantArgs a{};
    a.x = x; a.mat = matrix; a.col_major = matrix_col_major; a.f_out = out; a.M = M;
    a.table = matrix; a.n_table = 0;
    return signs_only ? launch_rows<fq::QM_PROJECT_SIGN>(a, x_dtype, D, stream)
                      : launch_rows<fq::QM_PROJECT>(a, x_dtype, D, stream);
}
