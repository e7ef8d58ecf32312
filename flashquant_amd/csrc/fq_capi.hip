// Library identification, status text and per-thread HIP error text of the C ABI.

#include <string>

#include "fq_common.hpp"

namespace {
thread_local std::string g_last_hip_error;
}

namespace fq_host {
void note_hip_error(hipError_t e) {
    g_last_hip_error = std::string(hipGetErrorName(e)) + ": " + hipGetErrorString(e);
}
}  // namespace fq_host

extern "C" int fq_abi_version(void) { return FQ_ABI_VERSION; }

extern "C" const char* fq_last_hip_error(void) { return g_last_hip_error.c_str(); }

extern "C" const char* fq_status_string(int status) {
    switch (status) {
        case FQ_OK: return "ok";
        case FQ_ERR_NULL_POINTER: return "a required pointer argument is NULL";
        case FQ_ERR_UNSUPPORTED_DIM: return "unsupported head_dim (must be 64, 128 or 256)";
        case FQ_ERR_UNSUPPORTED_BLOCK: return "unsupported block_size (must be 8, 16 or 32)";
        case FQ_ERR_UNSUPPORTED_DTYPE: return "unsupported dtype for this entry point";
        case FQ_ERR_BAD_SHAPE: return "bad shape argument";
        case FQ_ERR_MISALIGNED: return "pointer or stride not aligned as required";
        case FQ_ERR_WORKSPACE: return "workspace missing or too small";
        case FQ_ERR_LAUNCH: return "HIP runtime refused the launch";
        default: return "unknown status";
    }
}
