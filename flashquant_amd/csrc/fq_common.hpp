// Shared device/host helpers for the gfx950 TurboQuant kernels.
//
// Wavefronts are 64 lanes wide.  MFMA operand layouts used throughout:
//   v_mfma_f32_16x16x32_f16   A: lane l holds row l%16, k = 8*(l/16)+0..7
//                             B: lane l holds col l%16, k = 8*(l/16)+0..7
//                             C: lane l holds col l%16, rows 4*(l/16)+0..3
//   v_mfma_f32_32x32x16_f16   A: lane l holds row l%32, k = 8*(l/32)+0..7
//                             B: lane l holds col l%32, k = 8*(l/32)+0..7
//                             C: lane l holds col l%32, reg r <-> row 8*(r/4)+4*(l/32)+r%4
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/fq_hip.h"

namespace fq {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef _Float16 half2v __attribute__((ext_vector_type(2)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
typedef int int4v __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;

__device__ __forceinline__ float bits_to_float(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t float_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// bf16 <-> fp32.  The conversion to bf16 rounds to nearest even, as
// torch's Tensor.to(torch.bfloat16) does; NaN stays NaN.
__device__ __forceinline__ float bf16_to_float(uint16_t h) { return bits_to_float(uint32_t(h) << 16); }
__device__ __forceinline__ uint16_t float_to_bf16(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));   // v_cvt_pk_bf16_f32: round to nearest even
}
__device__ __forceinline__ float f16_to_float(uint16_t h) {
    return float(__builtin_bit_cast(_Float16, h));
}
__device__ __forceinline__ uint16_t float_to_f16(float f) {
    return __builtin_bit_cast(uint16_t, _Float16(f));  // v_cvt_f16_f32, round to nearest even
}

template <int DT> __device__ __forceinline__ float load_elem(uint16_t raw);
template <> __device__ __forceinline__ float load_elem<FQ_F16>(uint16_t raw) { return f16_to_float(raw); }
template <> __device__ __forceinline__ float load_elem<FQ_BF16>(uint16_t raw) { return bf16_to_float(raw); }
template <int DT> __device__ __forceinline__ uint16_t store_elem(float v);
template <> __device__ __forceinline__ uint16_t store_elem<FQ_F16>(float v) { return float_to_f16(v); }
template <> __device__ __forceinline__ uint16_t store_elem<FQ_BF16>(float v) { return float_to_bf16(v); }

typedef float float2v __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2v __attribute__((ext_vector_type(2)));

// two float32 values rounded to nearest even and packed, the first in the low half
// (v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32: one instruction per pair)
template <int DT> __device__ __forceinline__ uint32_t round_pair(float a, float b) {
    if constexpr (DT == FQ_BF16) return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{a, b}, bf16x2v));
    else return __builtin_bit_cast(uint32_t, __builtin_convertvector(float2v{a, b}, half2v));
}

__device__ __forceinline__ uint32_t pack_h2(_Float16 lo, _Float16 hi) {
    return uint32_t(__builtin_bit_cast(uint16_t, lo)) | (uint32_t(__builtin_bit_cast(uint16_t, hi)) << 16);
}

// Butterfly exchange with lane ^ mask inside the 64-lane wavefront.
__device__ __forceinline__ float xor_shuffle(float v, int mask) {
    return __shfl_xor(v, mask, kWave);
}

}  // namespace fq

// Host side: remember the last HIP error text per thread and map it to a status.
namespace fq_host {
void note_hip_error(hipError_t e);
inline int check_launch() {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        note_hip_error(e);
        return FQ_ERR_LAUNCH;
    }
    return FQ_OK;
}
inline bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }
inline bool supported_dim(int d) { return d == 64 || d == 128 || d == 256; }
// Raises the dynamic-LDS limit of a kernel function once per (function, device); later calls are a lookup.
bool lds_limit_raised(const void* kernel, size_t bytes);
int device_cu_count();
// Value of a kernel-variant switch (fq_option in fq_hip.h): its environment variable, read once
// per process, unless fq_set_option has changed it since.
int option(int id);
}  // namespace fq_host
