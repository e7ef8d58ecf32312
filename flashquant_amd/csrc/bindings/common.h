// Helpers shared by the pybind11 translation units of flashquant_amd._C.
#pragma once

#include <torch/extension.h>

#include <stdexcept>
#include <string>

#include "fq_hip.h"

namespace fqbind {

// C-ABI status -> Python exception.  Argument errors become ValueError (the
// reference's core raises std::invalid_argument for bad arguments,
// csrc/core/quantizer.cpp:13-18), runtime refusals become RuntimeError.
inline void raise_on_error(int status, const char* what) {
    if (status == FQ_OK) return;
    std::string msg = std::string(what) + ": " + fq_status_string(status);
    if (status == FQ_ERR_LAUNCH) {
        msg += " (";
        msg += fq_last_hip_error();
        msg += ")";
        throw std::runtime_error(msg);
    }
    throw std::invalid_argument(msg);
}

inline int dtype_code(at::ScalarType t, const char* what) {
    switch (t) {
        case at::kHalf: return FQ_F16;
        case at::kBFloat16: return FQ_BF16;
        case at::kFloat: return FQ_F32;
        default: throw std::invalid_argument(std::string(what) + ": dtype must be float16, bfloat16 or float32");
    }
}

inline void require_gpu(const at::Tensor& t, const char* name) {
    if (!t.is_cuda())
        throw std::invalid_argument(std::string(name) + " must live on the GPU (this module has no CPU path)");
}

inline void require(bool ok, const std::string& msg) {
    if (!ok) throw std::invalid_argument(msg);
}

void* current_stream(const at::Tensor& like);

}  // namespace fqbind

void bind_kernels(pybind11::module_& m);
void bind_codebook(pybind11::module_& m);
void bind_quantizer(pybind11::module_& m);
void bind_quantizer_classes(pybind11::module_& m);
