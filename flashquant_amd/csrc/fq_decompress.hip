// TQ4 decompress for gfx950: nibble unpack -> 16-entry centroid gather from
// LDS -> multiply by the row norm in float32 -> cast -> coalesced store.
//
// Pure streaming: 4 + D/2 bytes in, D * sizeof(out) bytes out per row.  One
// work unit is one packed dword (8 coordinates): a lane loads 4 bytes and
// stores 16 bytes (fp16/bf16) or 32 bytes (float32), so that a wavefront's
// loads and stores are each one contiguous span.  Output coordinate 2j comes
// from the high nibble of byte j and 2j+1 from the low nibble, as in
// decompress_reference (src/flashquant/kernels/cpu_reference.py:81-94).

#include "fq_common.hpp"

// The product centroid * norm must be rounded to float32 before it is rounded to
// the output type, as the reference does (two roundings).  Left alone, the
// compiler fuses the multiply and the fp16 conversion into one mixed-precision
// instruction (v_fma_mixlo_f16) with a single rounding, which differs from the
// reference on exact ties; the empty asm keeps the float32 product a value of
// its own.
__device__ __forceinline__ float rounded_product(float a, float b) {
    float p = a * b;
    asm volatile("" : "+v"(p));
    return p;
}

namespace fq {

constexpr int kDecThreads = 256;
constexpr int kDecUnroll = 8;   // packed dwords per lane: eight loads and eight 16-byte stores in flight

template <int DT>
__device__ __forceinline__ void store_unit(void* out, int64_t unit, const float (&v)[8]) {
    uint4v w;
    w.x = uint32_t(store_elem<DT>(v[0])) | (uint32_t(store_elem<DT>(v[1])) << 16);
    w.y = uint32_t(store_elem<DT>(v[2])) | (uint32_t(store_elem<DT>(v[3])) << 16);
    w.z = uint32_t(store_elem<DT>(v[4])) | (uint32_t(store_elem<DT>(v[5])) << 16);
    w.w = uint32_t(store_elem<DT>(v[6])) | (uint32_t(store_elem<DT>(v[7])) << 16);
    __builtin_nontemporal_store(w, reinterpret_cast<uint4v*>(out) + unit);
}
template <>
__device__ __forceinline__ void store_unit<FQ_F32>(void* out, int64_t unit, const float (&v)[8]) {
    float4v a = {v[0], v[1], v[2], v[3]};
    float4v b = {v[4], v[5], v[6], v[7]};
    float4v* p = reinterpret_cast<float4v*>(out) + unit * 2;
    __builtin_nontemporal_store(a, p);
    __builtin_nontemporal_store(b, p + 1);
}

// units_per_row_log2 = log2(D / 8)
template <int DT>
__global__ __launch_bounds__(kDecThreads) void tq4_decompress_kernel(
    const uint32_t* __restrict__ packed, const float* __restrict__ norms,
    const float* __restrict__ centroids, void* __restrict__ out,
    int64_t total_units, int units_per_row_log2) {
    __shared__ float lut[16];
    if (threadIdx.x < 16) lut[threadIdx.x] = centroids[threadIdx.x];
    __syncthreads();

    const int64_t base = (int64_t(blockIdx.x) * kDecUnroll) * kDecThreads + threadIdx.x;
    uint32_t word[kDecUnroll];
    float nrm[kDecUnroll];
#pragma unroll
    for (int u = 0; u < kDecUnroll; ++u) {
        const int64_t unit = base + int64_t(u) * kDecThreads;
        const bool live = unit < total_units;
        word[u] = live ? __builtin_nontemporal_load(packed + unit) : 0u;
        nrm[u] = live ? norms[unit >> units_per_row_log2] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < kDecUnroll; ++u) {
        const int64_t unit = base + int64_t(u) * kDecThreads;
        if (unit >= total_units) continue;
        float v[8];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            const uint32_t byte = (word[u] >> (8 * b)) & 0xffu;
            v[2 * b] = rounded_product(lut[byte >> 4], nrm[u]);
            v[2 * b + 1] = rounded_product(lut[byte & 15u], nrm[u]);
        }
        store_unit<DT>(out, unit, v);
    }
}

}  // namespace fq

extern "C" int fq_tq4_decompress(const uint8_t* packed, const float* norms,
                                 const float* centroids, void* out, int out_dtype,
                                 int64_t M, int D, void* stream) {
    using namespace fq;
    if (M < 0) return FQ_ERR_BAD_SHAPE;
    if (!fq_host::supported_dim(D)) return FQ_ERR_UNSUPPORTED_DIM;
    if (out_dtype != FQ_F16 && out_dtype != FQ_BF16 && out_dtype != FQ_F32) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (M == 0) return FQ_OK;
    if (!packed || !norms || !centroids || !out) return FQ_ERR_NULL_POINTER;
    if (!fq_host::aligned(packed, 4) || !fq_host::aligned(norms, 4) || !fq_host::aligned(out, 16))
        return FQ_ERR_MISALIGNED;

    const int log2_units = D == 64 ? 3 : (D == 128 ? 4 : 5);
    const int64_t total_units = M << log2_units;
    const int64_t per_block = int64_t(kDecThreads) * kDecUnroll;
    const int64_t blocks = (total_units + per_block - 1) / per_block;
    if (blocks > 0x7fffffffLL) return FQ_ERR_BAD_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t* pw = reinterpret_cast<const uint32_t*>(packed);
    dim3 grid(static_cast<unsigned>(blocks)), block(kDecThreads);
    switch (out_dtype) {
        case FQ_F16:
            hipLaunchKernelGGL(tq4_decompress_kernel<FQ_F16>, grid, block, 0, s, pw, norms, centroids, out, total_units, log2_units);
            break;
        case FQ_BF16:
            hipLaunchKernelGGL(tq4_decompress_kernel<FQ_BF16>, grid, block, 0, s, pw, norms, centroids, out, total_units, log2_units);
            break;
        default:
            hipLaunchKernelGGL(tq4_decompress_kernel<FQ_F32>, grid, block, 0, s, pw, norms, centroids, out, total_units, log2_units);
            break;
    }
    return fq_host::check_launch();
}
