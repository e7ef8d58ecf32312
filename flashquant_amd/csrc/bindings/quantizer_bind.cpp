// Set-up and quantizer bindings of flashquant_amd._C: the codebook solver, the seeded
// rotation and sketch matrices (host side, as in the reference), and the general
// TurboQuantMSE / TurboQuantProd row operators on the GPU.

#include <ATen/CPUGeneratorImpl.h>

#include <cmath>
#include <map>
#include <mutex>
#include <vector>

#include <pybind11/stl.h>

#include "common.h"

namespace py = pybind11;
using fqbind::require;

namespace {

// (centroids, boundaries) float32 on the CPU; the tuple the reference's Python layer
// unpacks from _C.codebook.solve_lloyd_max (src/flashquant/core/codebook.py:148-149).
std::tuple<at::Tensor, at::Tensor> solve_lloyd_max(int64_t dim, int64_t bits) {
    require(dim > 0, "dim must be positive");
    require(bits >= 1 && bits <= 8, "bits must lie in 1..8");
    at::Tensor c = at::empty({int64_t(1) << bits}, at::kFloat);
    at::Tensor b = at::empty({(int64_t(1) << bits) - 1}, at::kFloat);
    fqbind::raise_on_error(fq_lloyd_max_gaussian(int(dim), int(bits), c.data_ptr<float>(), b.data_ptr<float>()),
                           "solve_lloyd_max");
    return {c, b};
}

at::Tensor seeded_gaussian(int64_t rows, int64_t cols, int64_t seed) {
    auto gen = at::detail::createCPUGenerator(uint64_t(seed));
    return at::randn({rows, cols}, gen, at::TensorOptions().dtype(at::kFloat).device(at::kCPU));
}

// Haar rotation (src/flashquant/core/quantizer.py:60-85; csrc/core/rotation.cpp:8-39): QR of a
// seeded float32 Gaussian matrix on the CPU, the columns of Q multiplied by the sign of the
// diagonal of R with zero counted as +1.  The same library calls as the reference, so the same
// matrix on the same torch build.
at::Tensor haar_orthogonal(int64_t dim, int64_t seed) {
    require(dim > 0, "dim must be positive");
    const at::Tensor g = seeded_gaussian(dim, dim, seed);
    auto [q, r] = at::linalg_qr(g);
    at::Tensor s = at::sign(at::diagonal(r)).clone();
    s.masked_fill_(s == 0, 1.0);
    return q * s.unsqueeze(0);
}

// Sketch matrix of TurboQuantProd (src/flashquant/core/quantizer.py:264-268): generator seeded
// with seed + 1, divided by sqrt(qjl_dim).
at::Tensor qjl_matrix(int64_t dim, int64_t seed, std::optional<int64_t> qjl_dim) {
    const int64_t m = qjl_dim.value_or(dim);
    require(dim > 0 && m > 0, "dim and qjl_dim must be positive");
    return seeded_gaussian(m, dim, seed + 1) / std::sqrt(double(m));
}

// rotation.T[:, 0::2] and rotation.T[:, 1::2], contiguous (csrc/core/rotation.cpp:41-61).
std::tuple<at::Tensor, at::Tensor> split_rotation(const at::Tensor& rotation) {
    require(rotation.dim() == 2 && rotation.size(0) == rotation.size(1) && rotation.size(0) % 2 == 0,
            "rotation must be square with an even dimension");
    const at::Tensor rt = rotation.t().contiguous();
    using at::indexing::Slice;
    return {rt.index({Slice(), Slice(0, at::indexing::None, 2)}).contiguous(),
            rt.index({Slice(), Slice(1, at::indexing::None, 2)}).contiguous()};
}

struct MatArg {
    at::Tensor keep;
    int col_major = 0;
};
MatArg matrix_arg(const at::Tensor& mat, const c10::Device& dev, int64_t D, const char* name) {
    require(mat.dim() == 2 && mat.size(0) == D && mat.size(1) == D && mat.scalar_type() == at::kFloat,
            std::string(name) + " must be float32 of shape (D, D)");
    MatArg r;
    r.keep = mat.to(dev);
    if (!r.keep.is_contiguous()) {
        if (r.keep.t().is_contiguous()) r.col_major = 1;
        else r.keep = r.keep.contiguous();
    }
    return r;
}

at::Tensor float_rows(const at::Tensor& x, const char* name) {
    fqbind::require_gpu(x, name);
    require(x.dim() >= 1, std::string(name) + " must have a last dimension of head_dim");
    const auto t = x.scalar_type();
    if (t == at::kHalf || t == at::kBFloat16 || t == at::kFloat) return x.contiguous();
    return x.to(at::kFloat).contiguous();          // the reference casts every input with .float()
}

// TurboQuantMSE.quantize (src/flashquant/core/quantizer.py:125-157): (indices int64 (..., D),
// norms float32 (..., 1)).  `bits` is accepted for the reference's signature; the level count
// comes from the boundaries.
std::tuple<at::Tensor, at::Tensor> quantize(const at::Tensor& x, const at::Tensor& rotation,
                                            const at::Tensor& boundaries, int64_t bits) {
    const at::Tensor xc = float_rows(x, "x");
    const int64_t D = xc.size(-1), M = xc.numel() / (D > 0 ? D : 1);
    require(boundaries.scalar_type() == at::kFloat && boundaries.dim() == 1 && boundaries.numel() >= 1 &&
                boundaries.numel() <= 15,
            "boundaries must be 1 to 15 float32 values");
    require(bits <= 0 || boundaries.numel() == (int64_t(1) << bits) - 1, "boundaries must hold 2^bits - 1 values");
    c10::DeviceGuard guard(xc.device());
    const MatArg rot = matrix_arg(rotation, xc.device(), D, "rotation");
    const at::Tensor bd = boundaries.to(xc.device()).contiguous();
    at::Tensor idx = at::empty(xc.sizes(), xc.options().dtype(at::kLong));
    auto nshape = xc.sizes().vec();
    nshape.back() = 1;
    at::Tensor norms = at::empty(nshape, xc.options().dtype(at::kFloat));
    const int st = fq_mse_quantize(xc.data_ptr(), fqbind::dtype_code(xc.scalar_type(), "quantize"),
                                   rot.keep.data_ptr<float>(), rot.col_major, bd.data_ptr<float>(), int(bd.numel()),
                                   idx.data_ptr<int64_t>(), norms.data_ptr<float>(), M, int(D),
                                   fqbind::current_stream(xc));
    fqbind::raise_on_error(st, "quantize");
    return {idx, norms};
}

struct IdxArgs {
    at::Tensor idx, norms, cen;
    MatArg rot;
    int64_t M, D;
};
IdxArgs index_args(const at::Tensor& indices, const at::Tensor& norms, const at::Tensor& rotation,
                   const at::Tensor& centroids) {
    fqbind::require_gpu(indices, "indices");
    require(indices.dim() >= 1, "indices must have a last dimension of head_dim");
    IdxArgs a;
    a.idx = indices.to(at::kLong).contiguous();
    a.D = a.idx.size(-1);
    a.M = a.idx.numel() / (a.D > 0 ? a.D : 1);
    require(norms.numel() == a.M, "norms must hold one value per row");
    a.norms = norms.to(indices.device(), at::kFloat).contiguous();
    require(centroids.scalar_type() == at::kFloat && centroids.dim() == 1 && centroids.numel() >= 2 &&
                centroids.numel() <= 16,
            "centroids must be 2 to 16 float32 values");
    a.cen = centroids.to(indices.device()).contiguous();
    a.rot = matrix_arg(rotation, indices.device(), a.D, "rotation");
    return a;
}

// TurboQuantMSE.dequantize (src/flashquant/core/quantizer.py:159-195): float32, original space.
at::Tensor dequantize(const at::Tensor& indices, const at::Tensor& norms, const at::Tensor& rotation,
                      const at::Tensor& centroids) {
    c10::DeviceGuard guard(indices.device());
    const IdxArgs a = index_args(indices, norms, rotation, centroids);
    at::Tensor out = at::empty(a.idx.sizes(), a.idx.options().dtype(at::kFloat));
    const int st = fq_mse_dequantize(a.idx.data_ptr<int64_t>(), a.norms.data_ptr<float>(),
                                     a.rot.keep.data_ptr<float>(), a.rot.col_major, a.cen.data_ptr<float>(),
                                     int(a.cen.numel()), out.data_ptr<float>(), a.M, int(a.D),
                                     fqbind::current_stream(a.idx));
    fqbind::raise_on_error(st, "dequantize");
    return out;
}

// residual = x.float() - dequantize(indices, norms) and its row norms (..., 1)
// (src/flashquant/core/quantizer.py:290-295).
std::tuple<at::Tensor, at::Tensor> mse_residual(const at::Tensor& x, const at::Tensor& indices,
                                                const at::Tensor& norms, const at::Tensor& rotation,
                                                const at::Tensor& centroids) {
    const at::Tensor xc = float_rows(x, "x");
    c10::DeviceGuard guard(xc.device());
    const IdxArgs a = index_args(indices, norms, rotation, centroids);
    require(xc.sizes() == a.idx.sizes(), "x and indices must have one shape");
    at::Tensor res = at::empty(xc.sizes(), xc.options().dtype(at::kFloat));
    auto nshape = xc.sizes().vec();
    nshape.back() = 1;
    at::Tensor gam = at::empty(nshape, xc.options().dtype(at::kFloat));
    const int st = fq_mse_residual(xc.data_ptr(), fqbind::dtype_code(xc.scalar_type(), "mse_residual"),
                                   a.idx.data_ptr<int64_t>(), a.norms.data_ptr<float>(), a.rot.keep.data_ptr<float>(),
                                   a.rot.col_major, a.cen.data_ptr<float>(), int(a.cen.numel()), res.data_ptr<float>(),
                                   gam.data_ptr<float>(), a.M, int(a.D), fqbind::current_stream(xc));
    fqbind::raise_on_error(st, "mse_residual");
    return {res, gam};
}

// x @ matrix.T in float32, or its sign with 0 -> +1 (src/flashquant/core/quantizer.py:297-304, 357-359).
at::Tensor project_rows(const at::Tensor& x, const at::Tensor& matrix, bool signs_only) {
    const at::Tensor xc = float_rows(x, "x");
    const int64_t D = xc.size(-1), M = xc.numel() / (D > 0 ? D : 1);
    c10::DeviceGuard guard(xc.device());
    const MatArg mat = matrix_arg(matrix, xc.device(), D, "matrix");
    at::Tensor out = at::empty(xc.sizes(), xc.options().dtype(at::kFloat));
    const int st = fq_project_rows(xc.data_ptr(), fqbind::dtype_code(xc.scalar_type(), "project_rows"),
                                   mat.keep.data_ptr<float>(), mat.col_major, signs_only ? 1 : 0, out.data_ptr<float>(),
                                   M, int(D), fqbind::current_stream(xc));
    fqbind::raise_on_error(st, "project_rows");
    return out;
}

// ---------------------------------------------------------------------------------------
// The class surface of the reference's C++ core (csrc/core/types.h:9-38, codebook.h:17-68,
// quantizer.h:14-80, bound in csrc/bindings/codebook_bind.cpp:11-49 and quantizer_bind.cpp:10-64),
// over this library's host set-up and GPU kernels: construction and the codebook live on the
// host, the vectors on the GPU.
// ---------------------------------------------------------------------------------------
struct LloydMaxCodebook {
    at::Tensor centroids;    // (2^bits,) float32
    at::Tensor boundaries;   // (2^bits - 1,) float32
    int dim = 0;
    int bits = 0;
};

LloydMaxCodebook make_codebook(int dim, int bits) {
    auto [c, b] = solve_lloyd_max(dim, bits);
    return LloydMaxCodebook{c, b, dim, bits};
}

// torch.bucketize(x, boundaries) and centroids[indices] (csrc/core/codebook.cpp, codebook_quantize /
// codebook_dequantize): plain tensor-library calls on whatever device the data is on.
at::Tensor codebook_quantize(const at::Tensor& x, const at::Tensor& boundaries) {
    return at::bucketize(x, boundaries.to(x.device()).contiguous());
}
at::Tensor codebook_dequantize(const at::Tensor& indices, const at::Tensor& centroids) {
    return centroids.to(indices.device()).index({indices.to(at::kLong)});
}

class CodebookRegistry {
public:
    static CodebookRegistry& instance() {
        static CodebookRegistry r;
        return r;
    }
    LloydMaxCodebook get(int dim, int bits, const c10::Device& device) {
        std::lock_guard<std::mutex> lock(mu_);
        const std::string key = std::to_string(dim) + ":" + std::to_string(bits) + ":" + device.str();
        auto it = cache_.find(key);
        if (it != cache_.end()) return it->second;
        LloydMaxCodebook cb = make_codebook(dim, bits);
        cb.centroids = cb.centroids.to(device);
        cb.boundaries = cb.boundaries.to(device);
        cache_.emplace(key, cb);
        return cb;
    }
    void warmup(const std::vector<int>& dims, const std::vector<int>& bits_options, const c10::Device& device) {
        for (int d : dims)
            for (int b : bits_options) get(d, b, device);
    }
    void clear() {
        std::lock_guard<std::mutex> lock(mu_);
        cache_.clear();
    }

private:
    std::mutex mu_;
    std::map<std::string, LloydMaxCodebook> cache_;
};

struct QuantizedMSE {
    at::Tensor indices;   // (..., dim) int64
    at::Tensor norms;     // (..., 1) float32
};
struct QuantizedProd {
    at::Tensor indices;          // (..., dim) int64
    at::Tensor norms;            // (..., 1) float32
    at::Tensor qjl_signs;        // (..., dim) int8, +-1
    at::Tensor residual_norms;   // (..., 1) float32
};

class TurboQuantMSE {
public:
    TurboQuantMSE(int dim, int bits, int64_t seed) : dim_(dim), bits_(bits) {
        require(dim > 0, "dim must be positive");
        require(bits >= 1 && bits <= 4, "bits must lie in 1..4");
        rotation_ = haar_orthogonal(dim, seed);
        codebook_ = make_codebook(dim, bits);
    }
    QuantizedMSE quantize(const at::Tensor& x) const {
        require(x.dim() >= 1 && x.size(-1) == dim_, "the last dimension of x must be dim");
        auto [idx, norms] = ::quantize(x, rotation_, codebook_.boundaries, bits_);
        return QuantizedMSE{idx, norms};
    }
    at::Tensor dequantize(const at::Tensor& indices, const at::Tensor& norms) const {
        return ::dequantize(indices, norms, rotation_, codebook_.centroids);
    }
    const at::Tensor& rotation() const { return rotation_; }
    const LloydMaxCodebook& codebook() const { return codebook_; }
    int dim() const { return dim_; }
    int bits() const { return bits_; }

private:
    int dim_, bits_;
    at::Tensor rotation_;        // (dim, dim) float32 on the CPU; moved to the data's device per call
    LloydMaxCodebook codebook_;
};

class TurboQuantProd {
public:
    TurboQuantProd(int dim, int bits, int64_t seed)
        : dim_(dim), bits_(bits), mse_(dim, bits >= 2 ? bits - 1 : 1, seed) {
        require(bits >= 2, "TurboQuantProd requires bits >= 2 (1 bit for QJL), got " + std::to_string(bits));
        sketch_ = qjl_matrix(dim, seed, std::nullopt);
    }
    // csrc/core/quantizer.cpp:99-139: (bits - 1)-bit indices and norms, the residual's norm, and the
    // signs of the sketched residual as int8
    QuantizedProd quantize(const at::Tensor& x) const {
        const QuantizedMSE q = mse_.quantize(x);
        auto [residual, gamma] = mse_residual(x, q.indices, q.norms, mse_.rotation(), mse_.codebook().centroids);
        const at::Tensor signs = project_rows(residual, sketch_, true).to(at::kChar);
        return QuantizedProd{q.indices, q.norms, signs, gamma};
    }
    at::Tensor dequantize(const at::Tensor& indices, const at::Tensor& norms) const {
        return mse_.dequantize(indices, norms);
    }
    // <q, x_mse> + gamma sqrt(pi/2) / d <S q, signs>, one value per row (csrc/core/quantizer.cpp:148-184)
    at::Tensor estimate_inner_product(const at::Tensor& query, const QuantizedProd& c) const {
        require(query.dim() >= 1 && query.size(-1) == dim_, "the last dimension of query must be dim");
        const at::Tensor q2 = query.reshape({-1, dim_});
        const at::Tensor x_mse = mse_.dequantize(c.indices, c.norms).reshape({-1, dim_});
        const at::Tensor mse_term = at::sum(q2.to(at::kFloat) * x_mse, {-1}, true);
        const at::Tensor q_proj = project_rows(q2, sketch_, false);
        const at::Tensor dot = at::sum(q_proj * c.qjl_signs.reshape({-1, dim_}).to(at::kFloat), {-1}, true);
        const at::Tensor scale = c.residual_norms.reshape({-1, 1}) * (1.2533141373155003 / double(dim_));
        auto shape = query.sizes().vec();
        shape.back() = 1;
        return (mse_term + scale * dot).reshape(shape);
    }
    const TurboQuantMSE& mse_quantizer() const { return mse_; }
    const at::Tensor& sketch() const { return sketch_; }
    int dim() const { return dim_; }
    int bits() const { return bits_; }

private:
    int dim_, bits_;
    TurboQuantMSE mse_;
    at::Tensor sketch_;          // (dim, dim) float32 on the CPU
};

}  // namespace

void bind_codebook(py::module_& m) {
    py::module_ cb = m.def_submodule("codebook", "Lloyd-Max codebook (host)");
    // The two solvers return the (centroids, boundaries) tuple that the reference's Python layer
    // unpacks (src/flashquant/core/codebook.py:148-149), not the struct of the reference's C++.
    cb.def("solve_lloyd_max", &solve_lloyd_max, py::arg("dim"), py::arg("bits"),
           "(centroids, boundaries) float32 CPU tensors for N(0, 1/dim) truncated to +-3.5 sigma");
    cb.def("gaussian_lloyd_max", &solve_lloyd_max, py::arg("dim"), py::arg("bits"));
    py::class_<LloydMaxCodebook>(cb, "LloydMaxCodebook")
        .def(py::init(&make_codebook), py::arg("dim"), py::arg("bits"))
        .def_readwrite("centroids", &LloydMaxCodebook::centroids)
        .def_readwrite("boundaries", &LloydMaxCodebook::boundaries)
        .def_readonly("dim", &LloydMaxCodebook::dim)
        .def_readonly("bits", &LloydMaxCodebook::bits);
    cb.def("quantize", &codebook_quantize, py::arg("x"), py::arg("boundaries"),
           "Bucket index of every value: the number of boundaries below it");
    cb.def("dequantize", &codebook_dequantize, py::arg("indices"), py::arg("centroids"), "centroids[indices]");
    py::class_<CodebookRegistry>(cb, "CodebookRegistry")
        .def_static("instance", &CodebookRegistry::instance, py::return_value_policy::reference)
        .def("get", [](CodebookRegistry& self, int dim, int bits, c10::Device device) { return self.get(dim, bits, device); },
             py::arg("dim"), py::arg("bits"), py::arg("device"))
        .def("warmup", [](CodebookRegistry& self, const std::vector<int>& dims, const std::vector<int>& bits_options,
                          c10::Device device) { self.warmup(dims, bits_options, device); },
             py::arg("dims"), py::arg("bits_options"), py::arg("device"))
        .def("clear", &CodebookRegistry::clear);
}

void bind_quantizer_classes(py::module_& m) {
    py::module_ q = m.def_submodule("quantizer", "TurboQuant quantizers: set-up on the host, vectors on the GPU");
    py::class_<QuantizedMSE>(q, "QuantizedMSE")
        .def_readwrite("indices", &QuantizedMSE::indices)
        .def_readwrite("norms", &QuantizedMSE::norms);
    py::class_<QuantizedProd>(q, "QuantizedProd")
        .def_readwrite("indices", &QuantizedProd::indices)
        .def_readwrite("norms", &QuantizedProd::norms)
        .def_readwrite("qjl_signs", &QuantizedProd::qjl_signs)
        .def_readwrite("residual_norms", &QuantizedProd::residual_norms);
    py::class_<TurboQuantMSE>(q, "TurboQuantMSE")
        .def(py::init<int, int, int64_t>(), py::arg("dim"), py::arg("bits"), py::arg("seed") = 42)
        .def("quantize", &TurboQuantMSE::quantize, py::arg("x"), "QuantizedMSE(indices int64, norms float32) of GPU rows")
        .def("dequantize", &TurboQuantMSE::dequantize, py::arg("indices"), py::arg("norms"),
             "float32 rows in the original space")
        .def_property_readonly("dim", &TurboQuantMSE::dim)
        .def_property_readonly("bits", &TurboQuantMSE::bits)
        .def("rotation", [](const TurboQuantMSE& self) { return self.rotation(); })
        .def("codebook", [](const TurboQuantMSE& self) { return self.codebook(); });
    py::class_<TurboQuantProd>(q, "TurboQuantProd")
        .def(py::init<int, int, int64_t>(), py::arg("dim"), py::arg("bits"), py::arg("seed") = 42)
        .def("quantize", &TurboQuantProd::quantize, py::arg("x"), "QuantizedProd with int8 signs")
        .def("dequantize", &TurboQuantProd::dequantize, py::arg("indices"), py::arg("norms"),
             "Reconstruction from the (bits - 1)-bit stage alone")
        .def("estimate_inner_product", &TurboQuantProd::estimate_inner_product, py::arg("query"), py::arg("compressed"),
             "<q, x_mse> + gamma sqrt(pi/2) / d <S q, signs>, shape (..., 1)")
        .def_property_readonly("dim", &TurboQuantProd::dim)
        .def_property_readonly("bits", &TurboQuantProd::bits)
        .def("qjl_matrix", [](const TurboQuantProd& self) { return self.sketch(); });
}

void bind_quantizer(py::module_& m) {
    m.def("haar_orthogonal", &haar_orthogonal, py::arg("dim"), py::arg("seed") = 42,
          "Seeded Haar rotation, float32 (dim, dim) on the CPU");
    m.def("qjl_matrix", &qjl_matrix, py::arg("dim"), py::arg("seed") = 42, py::arg("qjl_dim") = py::none(),
          "Seeded Gaussian sketch / sqrt(qjl_dim), float32 (qjl_dim, dim) on the CPU");
    m.def("split_rotation", &split_rotation, py::arg("rotation"), "(rotation.T[:, 0::2], rotation.T[:, 1::2]) contiguous");
    // Not exported as `quantize` / `dequantize`: the reference's quantizer classes call those two
    // names with CPU tensors and no device test once they exist
    // (src/flashquant/core/quantizer.py:140-143, 176-179), and these operators are GPU kernels.
    m.def("mse_quantize", &quantize, py::arg("x"), py::arg("rotation"), py::arg("boundaries"), py::arg("bits") = 0,
          "TurboQuantMSE.quantize on the GPU: (indices int64 (..., D), norms float32 (..., 1))");
    m.def("mse_dequantize", &dequantize, py::arg("indices"), py::arg("norms"), py::arg("rotation"), py::arg("centroids"),
          "TurboQuantMSE.dequantize on the GPU: float32 (..., D) in the original space");
    m.def("mse_residual", &mse_residual, py::arg("x"), py::arg("indices"), py::arg("norms"), py::arg("rotation"),
          py::arg("centroids"), "(x - dequantize(indices, norms), its row norms)");
    m.def("project_rows", &project_rows, py::arg("x"), py::arg("matrix"), py::arg("signs_only") = false,
          "x @ matrix.T in float32, or its sign with 0 -> +1");
}
