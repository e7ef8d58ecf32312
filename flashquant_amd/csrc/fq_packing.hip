// Nibble pack / unpack of 4-bit indices on the GPU (src/flashquant/core/packing.py:54-98,
// csrc/core/packing.cpp:21-46): byte j = idx[2j] << 4 | idx[2j+1]; unpack interleaves
// [high, low].  Pure streaming.  Pack also counts indices outside [0, 15], which the
// reference rejects (validate_indices, csrc/core/packing.cpp:8-19).
#include "fq_common.hpp"

namespace fq {

template <typename T>
__global__ __launch_bounds__(256) void nibble_pack_kernel(const T* __restrict__ idx, uint8_t* __restrict__ packed,
                                                          int64_t n_packed, int* __restrict__ bad) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    int wrong = 0;
    if (i < n_packed) {
        const int64_t a = int64_t(idx[2 * i]), b = int64_t(idx[2 * i + 1]);
        wrong = (a < 0 || a > 15 || b < 0 || b > 15) ? 1 : 0;
        packed[i] = uint8_t(((a & 15) << 4) | (b & 15));
    }
    if (__any(wrong) && (threadIdx.x & 63) == 0) atomicAdd(bad, 1);   // one count per wavefront with a bad index
}

__global__ __launch_bounds__(256) void nibble_unpack_kernel(const uint8_t* __restrict__ packed,
                                                            int64_t* __restrict__ out, int64_t n_packed) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i < n_packed) {
        const uint32_t byte = packed[i];
        out[2 * i] = int64_t(byte >> 4);
        out[2 * i + 1] = int64_t(byte & 15u);
    }
}

// Four 2-bit indices per byte, the first in the top bits (csrc/core/packing.cpp:48-79).
template <typename T>
__global__ __launch_bounds__(256) void pack_2bit_kernel(const T* __restrict__ idx, uint8_t* __restrict__ packed,
                                                        int64_t n_packed, int* __restrict__ bad) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    int wrong = 0;
    if (i < n_packed) {
        uint32_t byte = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int64_t v = int64_t(idx[4 * i + k]);
            wrong |= (v < 0 || v > 3) ? 1 : 0;
            byte |= uint32_t(v & 3) << (6 - 2 * k);
        }
        packed[i] = uint8_t(byte);
    }
    if (__any(wrong) && (threadIdx.x & 63) == 0) atomicAdd(bad, 1);
}

__global__ __launch_bounds__(256) void unpack_2bit_kernel(const uint8_t* __restrict__ packed,
                                                          int64_t* __restrict__ out, int64_t n_packed) {
    const int64_t i = int64_t(blockIdx.x) * 256 + threadIdx.x;
    if (i < n_packed) {
        const uint32_t byte = packed[i];
#pragma unroll
        for (int k = 0; k < 4; ++k) out[4 * i + k] = int64_t((byte >> (6 - 2 * k)) & 3u);
    }
}

}  // namespace fq

extern "C" int fq_pack_2bit(const void* indices, int index_bytes, uint8_t* packed, int64_t n_packed,
                            int* bad_count, void* stream) {
    using namespace fq;
    if (n_packed < 0) return FQ_ERR_BAD_SHAPE;
    if (index_bytes != 1 && index_bytes != 4 && index_bytes != 8) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (n_packed == 0) return FQ_OK;
    if (!indices || !packed || !bad_count) return FQ_ERR_NULL_POINTER;
    const int64_t blocks = (n_packed + 255) / 256;
    if (blocks > 0x7fffffffLL) return FQ_ERR_BAD_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    if (index_bytes == 1)
        hipLaunchKernelGGL(pack_2bit_kernel<uint8_t>, grid, block, 0, s, static_cast<const uint8_t*>(indices), packed, n_packed, bad_count);
    else if (index_bytes == 4)
        hipLaunchKernelGGL(pack_2bit_kernel<int32_t>, grid, block, 0, s, static_cast<const int32_t*>(indices), packed, n_packed, bad_count);
    else
        hipLaunchKernelGGL(pack_2bit_kernel<int64_t>, grid, block, 0, s, static_cast<const int64_t*>(indices), packed, n_packed, bad_count);
    return fq_host::check_launch();
}

extern "C" int fq_unpack_2bit(const uint8_t* packed, int64_t* indices, int64_t n_packed, void* stream) {
    using namespace fq;
    if (n_packed < 0) return FQ_ERR_BAD_SHAPE;
    if (n_packed == 0) return FQ_OK;
    if (!packed || !indices) return FQ_ERR_NULL_POINTER;
    const int64_t blocks = (n_packed + 255) / 256;
    if (blocks > 0x7fffffffLL) return FQ_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(unpack_2bit_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), packed, indices, n_packed);
    return fq_host::check_launch();
}

extern "C" int fq_nibble_pack(const void* indices, int index_bytes, uint8_t* packed, int64_t n_packed,
                              int* bad_count, void* stream) {
    using namespace fq;
    if (n_packed < 0) return FQ_ERR_BAD_SHAPE;
    if (index_bytes != 1 && index_bytes != 4 && index_bytes != 8) return FQ_ERR_UNSUPPORTED_DTYPE;
    if (n_packed == 0) return FQ_OK;
    if (!indices || !packed || !bad_count) return FQ_ERR_NULL_POINTER;
    const int64_t blocks = (n_packed + 255) / 256;
    if (blocks > 0x7fffffffLL) return FQ_ERR_BAD_SHAPE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const dim3 grid(static_cast<unsigned>(blocks)), block(256);
    if (index_bytes == 1)
        hipLaunchKernelGGL(nibble_pack_kernel<uint8_t>, grid, block, 0, s, static_cast<const uint8_t*>(indices), packed, n_packed, bad_count);
    else if (index_bytes == 4)
        hipLaunchKernelGGL(nibble_pack_kernel<int32_t>, grid, block, 0, s, static_cast<const int32_t*>(indices), packed, n_packed, bad_count);
    else
        hipLaunchKernelGGL(nibble_pack_kernel<int64_t>, grid, block, 0, s, static_cast<const int64_t*>(indices), packed, n_packed, bad_count);
    return fq_host::check_launch();
}

extern "C" int fq_nibble_unpack(const uint8_t* packed, int64_t* indices, int64_t n_packed, void* stream) {
    using namespace fq;
    if (n_packed < 0) return FQ_ERR_BAD_SHAPE;
    if (n_packed == 0) return FQ_OK;
    if (!packed || !indices) return FQ_ERR_NULL_POINTER;
    const int64_t blocks = (n_packed + 255) / 256;
    if (blocks > 0x7fffffffLL) return FQ_ERR_BAD_SHAPE;
    hipLaunchKernelGGL(nibble_unpack_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), packed, indices, n_packed);
    return fq_host::check_launch();
}
