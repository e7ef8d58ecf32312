// Library identification, status text and per-thread HIP error text of the C ABI.

#include <atomic>
#include <cstdlib>
#include <mutex>
#include <string>

#include "fq_common.hpp"

namespace {
thread_local std::string g_last_hip_error;

// Kernel-variant switches: each takes its first value from an environment variable, read once
// per process, and can be changed afterwards with fq_set_option.
std::atomic<int> g_options[FQ_OPTION_COUNT];
std::once_flag g_options_once;
void init_options() {
    std::call_once(g_options_once, [] {
        const char* v = std::getenv("FQ_DECODE_COPY_WAVES");
        g_options[FQ_OPT_DECODE_COPY_WAVES] = (v != nullptr && v[0] == '0') ? 0 : 1;
        v = std::getenv("FQ_DECODE_DIRECT");
        g_options[FQ_OPT_DECODE_DIRECT] = (v != nullptr && v[0] == '1') ? 1 : 0;
        v = std::getenv("FQ_ATTENTION_ANY_DIM");
        g_options[FQ_OPT_ATTENTION_ANY_DIM] = (v != nullptr && v[0] == '1') ? 1 : 0;
        g_options[FQ_OPT_DECODE_TINY_SPIN] = 0;
        v = std::getenv("FQ_COMPRESS_THREE_TERMS");
        g_options[FQ_OPT_COMPRESS_THREE_TERMS] = (v != nullptr && v[0] == '1') ? 1 : 0;
        v = std::getenv("FQ_REDUCE_ROWS");
        g_options[FQ_OPT_REDUCE_ROWS] = v != nullptr ? std::atoi(v) : 0;
        v = std::getenv("FQ_DECODE_RING");
        g_options[FQ_OPT_DECODE_RING] = (v != nullptr && v[0] == '1') ? 1 : 0;
    });
}
}  // namespace

namespace fq_host {
void note_hip_error(hipError_t e) {
    g_last_hip_error = std::string(hipGetErrorName(e)) + ": " + hipGetErrorString(e);
}
int option(int id) {
    init_options();
    return g_options[id].load(std::memory_order_relaxed);
}
}  // namespace fq_host

extern "C" int fq_get_option(int option) {
    if (option < 0 || option >= FQ_OPTION_COUNT) return -1;
    return fq_host::option(option);
}

extern "C" int fq_set_option(int option, int value) {
    if (option < 0 || option >= FQ_OPTION_COUNT) return FQ_ERR_BAD_SHAPE;
    init_options();
    g_options[option].store(option == FQ_OPT_REDUCE_ROWS ? value : (value != 0 ? 1 : 0), std::memory_order_relaxed);
    return FQ_OK;
}

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
