// TQ4 decompress with the inverse rotation, one launch, gfx950.
//
// What the serving path does in two steps when it materialises the cache
// (_decompress_cache, src/flashquant/vllm/impl.py:265-318): tq4_decompress to the compute
// dtype (decompress_reference, src/flashquant/kernels/cpu_reference.py:64-94, cast at
// src/flashquant/kernels/decompress.py:80-81), then (x.float() @ rotation).to(dtype)
// (impl.py:309-316).  Per row:
//
//   v_j   = dtype(float32(centroid[idx_j] * norm))          rotated space, two roundings
//   out_i = dtype(sum_j float32(v_j) * R[j][i])             original space
//
// Bytes per row: 4 + D/2 in, 2 D out: the kernel is bound by HBM like the plain decompress,
// provided the contraction stays in the shadow of the memory traffic.  The v_j are 16-bit
// values by construction, so they go to the 32x32x16 MFMA of their own type exactly; R is
// stationary in registers as the A operand in two 16-bit terms (bf16: R = t0 + t1 to 2^-17,
// fp16: R = hi + lo / 4096 to 2^-22), which is far below the 2^-9 / 2^-12 rounding of the
// result.  A tile of 64 rows is dequantised into LDS (the B operand), each wavefront produces
// 32 output coordinates of every row, a lane ends with 16 consecutive coordinates of one row
// (the MFMA row index is permuted on the R side), and the rows leave through LDS in full
// 16-byte-per-lane spans.

#include "fq_common.hpp"

namespace fq {

namespace {

template <int D>
struct DecRotCfg {
    static constexpr int NK = D / 16;                  // MFMA k-steps
    static constexpr int CB = D / 32;                  // 32-coordinate output blocks
    static constexpr int WAVES = CB < 4 ? 4 : CB;
    static constexpr int THREADS = WAVES * kWave;
    static constexpr int TT = D == 256 ? 32 : 64;      // rows per tile
    static constexpr int TB = TT / 32;                 // 32-row blocks per tile
    static constexpr int TB_STEP = WAVES / CB;         // row blocks handled in parallel
    static constexpr int UPR = D / 8;                  // packed dwords (8 coordinates) per row
    static constexpr int UNITS = TT * UPR;             // per tile
    static constexpr int UPT = UNITS / THREADS;        // per thread
    static constexpr int STRIDE = D * 2 + 16;          // bytes per 16-bit row in LDS (padded)
};

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float two_roundings(float c, float n) {
    float p = c * n;                       // float32 product first, as the reference rounds it
    asm("" : "+v"(p));                     // (keeps the compiler from fusing it into the 16-bit conversion;
    return p;                              // not volatile: the products of a row may be scheduled freely)
}

// MFMA row r of a 32-row block <-> output coordinate (within the block) such that accumulator
// register i of lane half h holds coordinate 16 h + i.
__device__ __forceinline__ int row_to_coord(int r) { return 16 * ((r >> 2) & 1) + 4 * (r >> 3) + (r & 3); }

template <int D, int DT>
__global__ __launch_bounds__(DecRotCfg<D>::THREADS) void tq4_decompress_rotate_kernel(
    const uint32_t* __restrict__ packed, const float* __restrict__ norms, const float* __restrict__ centroids,
    const float* __restrict__ rotation, int col_major, uint16_t* __restrict__ out, int64_t M, int64_t num_tiles) {
    using C = DecRotCfg<D>;
    __shared__ __attribute__((aligned(16))) uint8_t xs[2][C::TT * C::STRIDE];   // dequantised rows, 16-bit
    __shared__ __attribute__((aligned(16))) uint8_t os[C::TT * C::STRIDE];      // rotated rows, 16-bit
    __shared__ float lut[16];

    const int tid = threadIdx.x;
    const int wave = tid / kWave, lane = tid % kWave;
    const int n32 = lane % 32, kg = lane / 32;
    const int cb = wave % C::CB, tb0 = wave / C::CB;

    if (tid < 16) lut[tid] = centroids[tid];

    // ---- the matrix rows of this wavefront: A[j][k] = R[k][j], two 16-bit terms ---------------
    constexpr bool kBf16 = DT == FQ_BF16;
    half8 a_hi[kBf16 ? 1 : C::NK], a_lo[kBf16 ? 1 : C::NK];
    bf16x8 a_t[kBf16 ? 2 : 1][kBf16 ? C::NK : 1];
    {
        const int j = 32 * cb + row_to_coord(n32);
#pragma unroll
        for (int ks = 0; ks < C::NK; ++ks)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int k = 16 * ks + 8 * kg + e;
                const float r = col_major ? rotation[k + int64_t(j) * D] : rotation[int64_t(k) * D + j];
                if constexpr (kBf16) {
                    const uint16_t t0 = float_to_bf16(r);
                    const uint16_t t1 = float_to_bf16(r - bf16_to_float(t0));
                    a_t[0][ks][e] = __builtin_bit_cast(__bf16, t0);
                    a_t[1][ks][e] = __builtin_bit_cast(__bf16, t1);
                } else {
                    const _Float16 hi = _Float16(r);
                    a_hi[ks][e] = hi;
                    a_lo[ks][e] = _Float16((r - float(hi)) * 4096.0f);
                }
            }
    }
    __syncthreads();

    // ---- staging: unit u of a tile = packed dword u % UPR of tile row u / UPR ------------------
    uint32_t word[C::UPT];
    float nrm[C::UPT];
    auto issue_loads = [&](int64_t tile) {
        if ((tile + 1) * C::TT <= M) {          // uniform: a whole tile needs no per-row conditions
            const uint32_t* src = packed + tile * C::TT * C::UPR;
            const float* nsrc = norms + tile * C::TT;
#pragma unroll
            for (int i = 0; i < C::UPT; ++i) {
                const int u = tid + i * C::THREADS;
                word[i] = __builtin_nontemporal_load(src + u);
                nrm[i] = nsrc[u / C::UPR];
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < C::UPT; ++i) {
            const int u = tid + i * C::THREADS;
            const int64_t row = tile * C::TT + u / C::UPR;
            const bool live = row < M;
            word[i] = live ? __builtin_nontemporal_load(packed + row * C::UPR + u % C::UPR) : 0u;
            nrm[i] = live ? norms[row] : 0.0f;
        }
    };
    auto stage = [&](int buf) {
#pragma unroll
        for (int i = 0; i < C::UPT; ++i) {
            const int u = tid + i * C::THREADS;
            uint32_t h[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const uint32_t byte = (word[i] >> (8 * b)) & 0xffu;
                h[b] = round_pair<DT>(two_roundings(lut[byte >> 4], nrm[i]), two_roundings(lut[byte & 15u], nrm[i]));
            }
            *reinterpret_cast<uint4v*>(&xs[buf][(u / C::UPR) * C::STRIDE + (u % C::UPR) * 16]) = uint4v{h[0], h[1], h[2], h[3]};
        }
    };
    auto store_tile = [&](int64_t tile) {
        constexpr int OC = D / 8;            // 16-byte chunks per output row
        for (int c = tid; c < C::TT * OC; c += C::THREADS) {
            const int r = c / OC, q = c % OC;
            const int64_t row = tile * C::TT + r;
            if (row < M) {
                const uint4v v = *reinterpret_cast<const uint4v*>(&os[r * C::STRIDE + q * 16]);
                __builtin_nontemporal_store(v, reinterpret_cast<uint4v*>(out + row * D) + q);
            }
        }
    };

    int64_t tile = blockIdx.x;
    if (tile < num_tiles) {
        issue_loads(tile);
        stage(0);
    }
    __syncthreads();
    for (int it = 0; tile < num_tiles; tile += gridDim.x, ++it) {
        const int cur = it & 1;
        const int64_t next = tile + gridDim.x;
        if (next < num_tiles) issue_loads(next);

        for (int tb = tb0; tb < C::TB; tb += C::TB_STEP) {
            const uint8_t* brow = &xs[cur][(32 * tb + n32) * C::STRIDE + kg * 16];
            float16v acc = {};
            float16v acc_lo = {};
            if constexpr (kBf16) {
#pragma unroll
                for (int t = 1; t >= 0; --t)          // the small term first
#pragma unroll
                    for (int ks = 0; ks < C::NK; ++ks) {
                        const bf16x8 b = *reinterpret_cast<const bf16x8*>(brow + ks * 32);
                        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a_t[t][ks], b, acc, 0, 0, 0);
                    }
            } else {
#pragma unroll
                for (int ks = 0; ks < C::NK; ++ks) {
                    const half8 b = *reinterpret_cast<const half8*>(brow + ks * 32);
                    acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_hi[ks], b, acc, 0, 0, 0);
                    acc_lo = __builtin_amdgcn_mfma_f32_32x32x16_f16(a_lo[ks], b, acc_lo, 0, 0, 0);
                }
            }
            uint32_t w[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float v0 = acc[2 * i], v1 = acc[2 * i + 1];
                if constexpr (!kBf16) {
                    v0 = __builtin_fmaf(acc_lo[2 * i], 1.0f / 4096.0f, v0);
                    v1 = __builtin_fmaf(acc_lo[2 * i + 1], 1.0f / 4096.0f, v1);
                }
                w[i] = round_pair<DT>(v0, v1);
            }
            uint8_t* dst = &os[(32 * tb + n32) * C::STRIDE + (32 * cb + 16 * kg) * 2];
            *reinterpret_cast<uint4v*>(dst) = uint4v{w[0], w[1], w[2], w[3]};
            *reinterpret_cast<uint4v*>(dst + 16) = uint4v{w[4], w[5], w[6], w[7]};
        }
        __syncthreads();                       // the rotated rows of this tile are complete
        store_tile(tile);
        if (next < num_tiles) stage(cur ^ 1);
        __syncthreads();                       // the next tile is staged; `os` is free again
    }
}

template <int D, int DT>
int launch_decompress_rotate(const uint8_t* packed, const float* norms, const float* centroids, const float* rotation,
                             int col_major, void* out, int64_t M, hipStream_t s) {
    using C = DecRotCfg<D>;
    const int64_t tiles = (M + C::TT - 1) / C::TT;
    // workgroups per CU: three fit the LDS at head_dim <= 128; the fp16 route holds two
    // accumulators per wavefront and runs faster with two
    const int64_t cap = int64_t(fq_host::device_cu_count()) * ((D == 256 || DT == FQ_F16) ? 2 : 3);
    const unsigned grid = unsigned(tiles < cap ? tiles : cap);
    hipLaunchKernelGGL((tq4_decompress_rotate_kernel<D, DT>), dim3(grid), dim3(C::THREADS), 0, s,
                       reinterpret_cast<const uint32_t*>(packed), norms, centroids, rotation, col_major,
                       static_cast<uint16_t*>(out), M, tiles);
    return fq_host::check_launch();
}

}  // namespace
}  // namespace fq

extern "C" int fq_tq4_decompress_rotated(const uint8_t* packed, const float* norms, const float* centroids,
                                         const float* rotation, int rotation_col_major, void* out, int out_dtype,
                                         int64_t M, int D, void* stream) {
    using namespace fq;
    if (M < 0) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (out_dtype != FQ_F16 && out_dtype != FQ_BF16) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (M == 0) return FQ_OK;
    if (!packed || !norms || !centroids || !rotation || !out) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(packed, 4) || !fq_host::aligned(norms, 4) || !fq_host::aligned(rotation, 4) ||
        !fq_host::aligned(out, 16))
        return FQ_ERR_MISALIGNED;
    hipStream_t s = static_cast<hipStream_t>(stream);
#define FQ_DECROT_CASE(DD)                                                                                          \
    case DD:                                                                                                        \
        return out_dtype == FQ_F16                                                                                  \
                   ? launch_decompress_rotate<DD, FQ_F16>(packed, norms, centroids, rotation, rotation_col_major, out, M, s) \
                   : launch_decompress_rotate<DD, FQ_BF16>(packed, norms, centroids, rotation, rotation_col_major, out, M, s);
    switch (D) {
        FQ_DECROT_CASE(64)
        FQ_DECROT_CASE(128)
        FQ_DECROT_CASE(256)
        default: return FQ_ERR_UNSUPPORTED_DIM;
    }
#undef FQ_DECROT_CASE
}
