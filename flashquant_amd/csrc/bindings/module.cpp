// flashquant_amd._C: pybind11 module over libfq_hip.so.  Built so that the same
// shared object can be installed as flashquant._C: the module name is "_C" and
// the attribute names are the ones the reference's Python layer probes for.

#include "common.h"

namespace py = pybind11;

PYBIND11_MODULE(_C, m) {
    m.doc() = "TurboQuant KV-cache kernels for MI355X (gfx950)";
    m.attr("abi_version") = fq_abi_version();
    bind_kernels(m);
    bind_codebook(m);
    bind_quantizer(m);
    bind_quantizer_classes(m);
}
