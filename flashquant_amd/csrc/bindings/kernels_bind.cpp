// Kernel bindings of flashquant_amd._C: the operator names and argument orders
// that the reference's Python dispatch layer probes for with hasattr(_C, ...)
// and calls (src/flashquant/kernels/compress.py:90-92, decompress.py:77,
// paged_decode.py:105-110, src/flashquant/vllm/impl.py:380-393).  Each function
// unwraps torch tensors and calls the C ABI of libfq_hip.so on torch's current
// stream.  There is no CPU path: a tensor that is not on the GPU is an error.

#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>

#include <optional>
#include <tuple>

#include "common.h"

namespace py = pybind11;
using fqbind::require;

namespace fqbind {
void* current_stream(const at::Tensor& like) {
    return static_cast<void*>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(like.device().index()).stream());
}
}  // namespace fqbind

namespace {

// A (D, D) float32 rotation on the right device as the C ABI wants it: row-major, or
// column-major when the transpose is the contiguous one (no copy in either case).
struct RotationArg {
    at::Tensor keep;
    const float* ptr = nullptr;
    int col_major = 0;
};
RotationArg rotation_arg(const at::Tensor& rotation, const c10::Device& dev, int64_t D) {
    require(rotation.dim() == 2 && rotation.size(0) == D && rotation.size(1) == D && rotation.scalar_type() == at::kFloat,
            "rotation must be float32 of shape (D, D)");
    RotationArg r;
    r.keep = rotation.to(dev);
    if (!r.keep.is_contiguous()) {
        if (r.keep.t().is_contiguous()) r.col_major = 1;
        else r.keep = r.keep.contiguous();
    }
    r.ptr = r.keep.data_ptr<float>();
    return r;
}

int option_id(const std::string& name) {
    if (name == "decode_copy_waves") return FQ_OPT_DECODE_COPY_WAVES;
    if (name == "decode_direct") return FQ_OPT_DECODE_DIRECT;
    if (name == "attention_any_dim") return FQ_OPT_ATTENTION_ANY_DIM;
    if (name == "decode_tiny_spin") return FQ_OPT_DECODE_TINY_SPIN;
    if (name == "compress_three_terms") return FQ_OPT_COMPRESS_THREE_TERMS;
    if (name == "decode_ring") return FQ_OPT_DECODE_RING;
    if (name == "reduce_rows") return FQ_OPT_REDUCE_ROWS;
    throw std::invalid_argument("unknown option '" + name + "'");
}

using OptPair = std::optional<std::tuple<at::Tensor, at::Tensor>>;

std::tuple<at::Tensor, at::Tensor> tq4_compress(const at::Tensor& x, const at::Tensor& rot_T_even,
                                                const at::Tensor& rot_T_odd, const at::Tensor& boundaries,
                                                const OptPair& out) {
    fqbind::require_gpu(x, "x");
    require(x.dim() == 3, "x must have shape (N, H, D)");
    const int64_t N = x.size(0), H = x.size(1), D = x.size(2);
    require(x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16,
            "tq4_compress: x must be float16 or bfloat16 on the GPU");
    require(rot_T_even.scalar_type() == at::kFloat && rot_T_odd.scalar_type() == at::kFloat &&
                boundaries.scalar_type() == at::kFloat,
            "rotation halves and boundaries must be float32");
    require(rot_T_even.dim() == 2 && rot_T_even.size(0) == D && rot_T_even.size(1) == D / 2 &&
                rot_T_odd.sizes() == rot_T_even.sizes(),
            "rotation halves must have shape (D, D/2)");
    require(boundaries.numel() == 15, "boundaries must hold 15 values (4-bit codebook)");
    c10::DeviceGuard guard(x.device());
    const at::Tensor xc = x.contiguous();
    const at::Tensor re = rot_T_even.to(x.device()).contiguous();
    const at::Tensor ro = rot_T_odd.to(x.device()).contiguous();
    const at::Tensor bd = boundaries.to(x.device()).contiguous();
    at::Tensor packed, norms;
    if (out.has_value()) {
        packed = std::get<0>(*out);
        norms = std::get<1>(*out);
        require(packed.is_cuda() && norms.is_cuda() && packed.is_contiguous() && norms.is_contiguous(),
                "out buffers must be contiguous GPU tensors");
        require(packed.scalar_type() == at::kByte && norms.scalar_type() == at::kFloat,
                "out must be (uint8 packed, float32 norms)");
        require(packed.numel() >= N * H * (D / 2) && norms.numel() >= N * H, "out buffers are too small");
        packed = packed.flatten().narrow(0, 0, N * H * (D / 2)).view({N, H, D / 2});
        norms = norms.flatten().narrow(0, 0, N * H).view({N, H, 1});
    } else {
        packed = at::empty({N, H, D / 2}, x.options().dtype(at::kByte));
        norms = at::empty({N, H, 1}, x.options().dtype(at::kFloat));
    }
    const int st = fq_tq4_compress(xc.data_ptr(), fqbind::dtype_code(x.scalar_type(), "tq4_compress"),
                                   re.data_ptr<float>(), ro.data_ptr<float>(), bd.data_ptr<float>(),
                                   packed.data_ptr<uint8_t>(), norms.data_ptr<float>(), N * H, int(D),
                                   fqbind::current_stream(x));
    fqbind::raise_on_error(st, "tq4_compress");
    return {packed, norms};
}

void tq4_compress_store(const at::Tensor& key, const at::Tensor& value, const at::Tensor& rot_T_even,
                        const at::Tensor& rot_T_odd, const at::Tensor& boundaries, at::Tensor kv_cache,
                        const at::Tensor& slot_mapping) {
    fqbind::require_gpu(key, "key");
    fqbind::require_gpu(value, "value");
    fqbind::require_gpu(kv_cache, "kv_cache");
    require(key.dim() == 3 && value.sizes() == key.sizes() && value.scalar_type() == key.scalar_type(),
            "key and value must both have shape (N, H, D) and one dtype");
    require(key.scalar_type() == at::kHalf || key.scalar_type() == at::kBFloat16, "key/value must be float16 or bfloat16");
    const int64_t N = key.size(0), H = key.size(1), D = key.size(2);
    require(rot_T_even.scalar_type() == at::kFloat && rot_T_odd.scalar_type() == at::kFloat &&
                boundaries.scalar_type() == at::kFloat,
            "rotation halves and boundaries must be float32");
    require(rot_T_even.dim() == 2 && rot_T_even.size(0) == D && rot_T_even.size(1) == D / 2 &&
                rot_T_odd.sizes() == rot_T_even.sizes(),
            "rotation halves must have shape (D, D/2)");
    require(boundaries.numel() == 15, "boundaries must hold 15 values (4-bit codebook)");
    require(kv_cache.scalar_type() == at::kByte && kv_cache.is_contiguous() && kv_cache.dim() >= 2 &&
                kv_cache.size(-1) == H * (D + 8),
            "kv_cache must be a contiguous uint8 tensor whose last dimension is H * (D + 8)");
    require(slot_mapping.dim() == 1 && slot_mapping.size(0) <= N, "slot_mapping must be 1-D with at most N entries");
    c10::DeviceGuard guard(key.device());
    const at::Tensor kc = key.contiguous(), vc = value.contiguous();
    const at::Tensor re = rot_T_even.to(key.device()).contiguous();
    const at::Tensor ro = rot_T_odd.to(key.device()).contiguous();
    const at::Tensor bd = boundaries.to(key.device()).contiguous();
    const at::Tensor sm = slot_mapping.to(key.device(), at::kLong).contiguous();
    const int64_t num_slots = kv_cache.numel() / (H * (D + 8));
    const int st = fq_tq4_compress_store(kc.data_ptr(), vc.data_ptr(), fqbind::dtype_code(key.scalar_type(), "tq4_compress_store"),
                                         re.data_ptr<float>(), ro.data_ptr<float>(), bd.data_ptr<float>(),
                                         kv_cache.data_ptr<uint8_t>(), sm.data_ptr<int64_t>(), N, sm.size(0), int(H),
                                         int(D), num_slots, fqbind::current_stream(key));
    fqbind::raise_on_error(st, "tq4_compress_store");
}

// tq4_decompress followed by (x.float() @ rotation).to(dtype), one launch
// (src/flashquant/vllm/impl.py:298-316).
at::Tensor tq4_decompress_rotated(const at::Tensor& packed, const at::Tensor& norms, const at::Tensor& centroids,
                                  const at::Tensor& rotation, at::ScalarType dtype,
                                  const std::optional<at::Tensor>& out) {
    fqbind::require_gpu(packed, "packed");
    require(packed.dim() == 3 && packed.scalar_type() == at::kByte, "packed must be uint8 of shape (N, H, D/2)");
    const int64_t N = packed.size(0), H = packed.size(1), D = 2 * packed.size(2);
    require(norms.scalar_type() == at::kFloat && norms.numel() == N * H, "norms must be float32 of shape (N, H, 1)");
    require(centroids.scalar_type() == at::kFloat && centroids.numel() == 16, "centroids must be 16 float32 values");
    require(dtype == at::kHalf || dtype == at::kBFloat16, "tq4_decompress_rotated: dtype must be float16 or bfloat16");
    c10::DeviceGuard guard(packed.device());
    const at::Tensor pc = packed.contiguous();
    const at::Tensor nc = norms.to(packed.device()).contiguous();
    const at::Tensor cc = centroids.to(packed.device()).contiguous();
    const RotationArg rot = rotation_arg(rotation, packed.device(), D);
    at::Tensor result;
    if (out.has_value()) {
        result = *out;
        require(result.is_cuda() && result.is_contiguous() && result.scalar_type() == dtype &&
                    result.numel() >= N * H * D,
                "out must be a contiguous GPU tensor of the requested dtype with room for (N, H, D)");
        result = result.flatten().narrow(0, 0, N * H * D).view({N, H, D});
    } else {
        result = at::empty({N, H, D}, packed.options().dtype(dtype));
    }
    const int st = fq_tq4_decompress_rotated(pc.data_ptr<uint8_t>(), nc.data_ptr<float>(), cc.data_ptr<float>(), rot.ptr,
                                             rot.col_major, result.data_ptr(),
                                             fqbind::dtype_code(dtype, "tq4_decompress_rotated"), N * H, int(D),
                                             fqbind::current_stream(packed));
    fqbind::raise_on_error(st, "tq4_decompress_rotated");
    return result;
}

at::Tensor tq4_decompress(const at::Tensor& packed, const at::Tensor& norms, const at::Tensor& centroids,
                          at::ScalarType dtype, const std::optional<at::Tensor>& out) {
    fqbind::require_gpu(packed, "packed");
    require(packed.dim() == 3 && packed.scalar_type() == at::kByte, "packed must be uint8 of shape (N, H, D/2)");
    const int64_t N = packed.size(0), H = packed.size(1), D = 2 * packed.size(2);
    require(norms.scalar_type() == at::kFloat && norms.numel() == N * H, "norms must be float32 of shape (N, H, 1)");
    require(centroids.scalar_type() == at::kFloat && centroids.numel() == 16, "centroids must be 16 float32 values");
    c10::DeviceGuard guard(packed.device());
    const at::Tensor pc = packed.contiguous();
    const at::Tensor nc = norms.to(packed.device()).contiguous();
    const at::Tensor cc = centroids.to(packed.device()).contiguous();
    at::Tensor result;
    if (out.has_value()) {
        result = *out;
        require(result.is_cuda() && result.is_contiguous() && result.scalar_type() == dtype &&
                    result.numel() >= N * H * D,
                "out must be a contiguous GPU tensor of the requested dtype with room for (N, H, D)");
        result = result.flatten().narrow(0, 0, N * H * D).view({N, H, D});
    } else {
        result = at::empty({N, H, D}, packed.options().dtype(dtype));
    }
    const int st = fq_tq4_decompress(pc.data_ptr<uint8_t>(), nc.data_ptr<float>(), cc.data_ptr<float>(),
                                     result.data_ptr(), fqbind::dtype_code(dtype, "tq4_decompress"), N * H, int(D),
                                     fqbind::current_stream(packed));
    fqbind::raise_on_error(st, "tq4_decompress");
    return result;
}

// The no-allocation variant: the binding converts and allocates nothing either, so every operand
// has to be on the GPU and contiguous already.
at::Tensor split_k_paged_decode_static(const at::Tensor& q, const at::Tensor& kv_cache, const at::Tensor& block_table,
                                       const at::Tensor& seq_lens, const at::Tensor& centroids_k,
                                       const at::Tensor& centroids_v, const std::optional<at::Tensor>& rotation,
                                       int64_t num_kv_heads, int64_t head_dim, int64_t block_size, double sm_scale,
                                       const at::Tensor& out, int64_t num_splits) {
    for (const at::Tensor* t : {&q, &kv_cache, &block_table, &seq_lens, &centroids_k, &centroids_v, &out}) {
        fqbind::require_gpu(*t, "every operand");
        require(t->is_contiguous(), "every operand must be contiguous");
    }
    require(q.dim() == 3 && q.size(2) == head_dim, "q must have shape (num_seqs, H_Q, D)");
    require(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "q must be float16 or bfloat16");
    require(kv_cache.dim() == 3 && kv_cache.scalar_type() == at::kByte && kv_cache.size(1) == block_size &&
                kv_cache.size(2) == num_kv_heads * (head_dim + 8),
            "kv_cache must be uint8 of shape (num_blocks, block_size, num_kv_heads * (head_dim + 8))");
    require(block_table.dim() == 2 && block_table.scalar_type() == at::kInt && block_table.size(0) == q.size(0),
            "block_table must be int32 of shape (num_seqs, max_blocks)");
    require(seq_lens.scalar_type() == at::kInt && seq_lens.numel() == q.size(0), "seq_lens must be int32 (num_seqs,)");
    require(centroids_k.numel() == 16 && centroids_v.numel() == 16 && centroids_k.scalar_type() == at::kFloat &&
                centroids_v.scalar_type() == at::kFloat,
            "centroids must be 16 float32 values");
    require(out.scalar_type() == q.scalar_type() && out.sizes() == q.sizes(), "out must have the shape and dtype of q");
    require(num_splits >= 0, "num_splits must be >= 0");
    const float* rot = nullptr;
    int col_major = 0;
    if (rotation.has_value()) {
        const at::Tensor& r = *rotation;
        fqbind::require_gpu(r, "rotation");
        require(r.dim() == 2 && r.size(0) == head_dim && r.size(1) == head_dim && r.scalar_type() == at::kFloat,
                "rotation must be float32 of shape (D, D)");
        require(r.is_contiguous() || r.t().is_contiguous(), "rotation must be contiguous, or the transpose of a contiguous matrix");
        col_major = r.is_contiguous() ? 0 : 1;
        rot = r.data_ptr<float>();
    }
    c10::DeviceGuard guard(q.device());
    const int st = fq_split_k_paged_decode_static(
        q.data_ptr(), kv_cache.data_ptr<uint8_t>(), block_table.data_ptr<int32_t>(), seq_lens.data_ptr<int32_t>(),
        centroids_k.data_ptr<float>(), centroids_v.data_ptr<float>(), rot, col_major, out.data_ptr(), int(q.size(0)),
        int(q.size(1)), int(num_kv_heads), int(head_dim), int(block_size), int(block_table.size(1)), kv_cache.size(0),
        float(sm_scale), fqbind::dtype_code(q.scalar_type(), "split_k_paged_decode_static"), int(num_splits),
        fqbind::current_stream(q));
    fqbind::raise_on_error(st, "split_k_paged_decode_static");
    return out;
}

at::Tensor split_k_paged_decode(const at::Tensor& q, const at::Tensor& kv_cache, const at::Tensor& block_table,
                                const at::Tensor& seq_lens, const at::Tensor& centroids_k,
                                const at::Tensor& centroids_v, const std::optional<at::Tensor>& rotation,
                                int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                                std::optional<double> sm_scale, const std::optional<at::Tensor>& out,
                                int64_t num_splits, const std::optional<at::Tensor>& workspace) {
    fqbind::require_gpu(q, "q");
    fqbind::require_gpu(kv_cache, "kv_cache");
    require(q.dim() == 3 && q.size(2) == head_dim, "q must have shape (num_seqs, H_Q, D)");
    require(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "q must be float16 or bfloat16");
    require(kv_cache.dim() == 3 && kv_cache.scalar_type() == at::kByte && kv_cache.is_contiguous(),
            "kv_cache must be a contiguous uint8 tensor (num_blocks, block_size, bytes)");
    require(kv_cache.size(1) == block_size && kv_cache.size(2) == num_kv_heads * (head_dim + 8),
            "kv_cache must have shape (num_blocks, block_size, num_kv_heads * (head_dim + 8))");
    require(block_table.dim() == 2 && block_table.scalar_type() == at::kInt && block_table.size(0) == q.size(0),
            "block_table must be int32 of shape (num_seqs, max_blocks)");
    require(seq_lens.scalar_type() == at::kInt && seq_lens.numel() == q.size(0), "seq_lens must be int32 (num_seqs,)");
    require(centroids_k.numel() == 16 && centroids_v.numel() == 16 && centroids_k.scalar_type() == at::kFloat &&
                centroids_v.scalar_type() == at::kFloat,
            "centroids must be 16 float32 values");
    require(num_splits >= 0, "num_splits must be >= 0");
    c10::DeviceGuard guard(q.device());
    const int S = int(q.size(0)), HQ = int(q.size(1)), D = int(head_dim);
    const double scale = sm_scale.has_value() ? *sm_scale : 1.0 / std::sqrt(double(head_dim));
    const at::Tensor qc = q.contiguous();
    const at::Tensor bt = block_table.to(q.device()).contiguous();
    const at::Tensor sl = seq_lens.to(q.device()).contiguous();
    const at::Tensor ck = centroids_k.to(q.device()).contiguous();
    const bool same = centroids_v.is_same(centroids_k) ||
                      (centroids_v.device() == centroids_k.device() && centroids_v.data_ptr() == centroids_k.data_ptr());
    const at::Tensor cv = same ? ck : centroids_v.to(q.device()).contiguous();
    RotationArg rot;
    if (rotation.has_value()) rot = rotation_arg(*rotation, q.device(), D);
    at::Tensor result;
    if (out.has_value()) {
        result = *out;
        require(result.is_cuda() && result.is_contiguous() && result.scalar_type() == q.scalar_type() &&
                    result.sizes() == q.sizes(),
                "out must be a contiguous GPU tensor with the shape and dtype of q");
    } else {
        result = at::empty_like(qc);
    }
    const int max_blocks = int(bt.size(1));
    const size_t ws_bytes = fq_paged_decode_workspace_bytes(S, HQ, int(num_kv_heads), D, int(block_size), max_blocks,
                                                            int(num_splits));
    at::Tensor ws;
    if (workspace.has_value()) {      // the caller's scratch (any contents): nothing is allocated for it here
        ws = *workspace;
        require(ws.is_cuda() && ws.device() == q.device() && ws.is_contiguous() && ws.scalar_type() == at::kByte &&
                    size_t(ws.numel()) >= ws_bytes,
                "workspace must be a contiguous uint8 GPU tensor of at least paged_decode_workspace_bytes(...) bytes");
    } else {
        ws = at::empty({int64_t(ws_bytes)}, q.options().dtype(at::kByte));
    }
    const int st = fq_split_k_paged_decode(
        qc.data_ptr(), kv_cache.data_ptr<uint8_t>(), bt.data_ptr<int32_t>(), sl.data_ptr<int32_t>(),
        ck.data_ptr<float>(), cv.data_ptr<float>(), rot.ptr, rot.col_major, result.data_ptr(),
        S, HQ, int(num_kv_heads), D, int(block_size), max_blocks, kv_cache.size(0), float(scale),
        fqbind::dtype_code(q.scalar_type(), "split_k_paged_decode"), int(num_splits), ws.data_ptr(), size_t(ws.numel()),
        fqbind::current_stream(q));
    fqbind::raise_on_error(st, "split_k_paged_decode");
    return result;
}

// One serving step (src/flashquant/vllm/impl.py:362-394): the new token of every sequence into its cache
// row, then the decode.  Everything must already be on the GPU (a serving loop's tensors are).
at::Tensor tq4_store_and_decode(const at::Tensor& key, const at::Tensor& value, const at::Tensor& slot_mapping,
                                const at::Tensor& rot_T_even, const at::Tensor& rot_T_odd, const at::Tensor& boundaries,
                                const at::Tensor& q, at::Tensor kv_cache, const at::Tensor& block_table,
                                const at::Tensor& seq_lens, const at::Tensor& centroids_k, const at::Tensor& centroids_v,
                                const at::Tensor& rotation, int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                                std::optional<double> sm_scale, const std::optional<at::Tensor>& out, int64_t num_splits,
                                const std::optional<at::Tensor>& workspace) {
    const at::Tensor& cache_ref = kv_cache;
    for (const at::Tensor* t : {&key, &value, &slot_mapping, &rot_T_even, &rot_T_odd, &boundaries, &q, &cache_ref,
                                &block_table, &seq_lens, &centroids_k, &centroids_v, &rotation})
        fqbind::require_gpu(*t, "every operand");
    require(q.dim() == 3 && q.size(2) == head_dim, "q must have shape (num_seqs, H_Q, D)");
    require(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "q must be float16 or bfloat16");
    const int64_t S = q.size(0), HQ = q.size(1), D = head_dim, H = num_kv_heads;
    require(key.dim() == 3 && key.size(0) == S && key.size(1) == H && key.size(2) == D && value.sizes() == key.sizes() &&
                key.scalar_type() == q.scalar_type() && value.scalar_type() == q.scalar_type(),
            "key and value must have shape (num_seqs, H_KV, D) and the dtype of q");
    require(slot_mapping.dim() == 1 && slot_mapping.size(0) == S && slot_mapping.scalar_type() == at::kLong,
            "slot_mapping must be int64 of shape (num_seqs,)");
    require(rot_T_even.scalar_type() == at::kFloat && rot_T_odd.scalar_type() == at::kFloat &&
                boundaries.scalar_type() == at::kFloat && rot_T_even.dim() == 2 && rot_T_even.size(0) == D &&
                rot_T_even.size(1) == D / 2 && rot_T_odd.sizes() == rot_T_even.sizes() && boundaries.numel() == 15,
            "rotation halves must be float32 (D, D/2), boundaries 15 float32 values");
    require(kv_cache.dim() == 3 && kv_cache.scalar_type() == at::kByte && kv_cache.is_contiguous() &&
                kv_cache.size(1) == block_size && kv_cache.size(2) == H * (D + 8),
            "kv_cache must be contiguous uint8 of shape (num_blocks, block_size, num_kv_heads * (head_dim + 8))");
    require(block_table.dim() == 2 && block_table.scalar_type() == at::kInt && block_table.size(0) == S,
            "block_table must be int32 of shape (num_seqs, max_blocks)");
    require(seq_lens.scalar_type() == at::kInt && seq_lens.numel() == S, "seq_lens must be int32 (num_seqs,)");
    require(centroids_k.numel() == 16 && centroids_v.numel() == 16 && centroids_k.scalar_type() == at::kFloat &&
                centroids_v.scalar_type() == at::kFloat,
            "centroids must be 16 float32 values");
    require(num_splits >= 0, "num_splits must be >= 0");
    c10::DeviceGuard guard(q.device());
    const double scale = sm_scale.has_value() ? *sm_scale : 1.0 / std::sqrt(double(head_dim));
    const at::Tensor kc = key.contiguous(), vc = value.contiguous(), qc = q.contiguous();
    const at::Tensor re = rot_T_even.contiguous(), ro = rot_T_odd.contiguous(), bd = boundaries.contiguous();
    const at::Tensor bt = block_table.contiguous(), sl = seq_lens.contiguous(), sm = slot_mapping.contiguous();
    const at::Tensor ck = centroids_k.contiguous();
    const bool same = centroids_v.is_same(centroids_k) || centroids_v.data_ptr() == centroids_k.data_ptr();
    const at::Tensor cv = same ? ck : centroids_v.contiguous();
    const RotationArg rot = rotation_arg(rotation, q.device(), int(D));
    at::Tensor result;
    if (out.has_value()) {
        result = *out;
        require(result.is_cuda() && result.is_contiguous() && result.scalar_type() == q.scalar_type() &&
                    result.sizes() == q.sizes(),
                "out must be a contiguous GPU tensor with the shape and dtype of q");
    } else {
        result = at::empty_like(qc);
    }
    const int max_blocks = int(bt.size(1));
    const size_t ws_bytes = fq_paged_decode_workspace_bytes(int(S), int(HQ), int(H), int(D), int(block_size), max_blocks,
                                                            int(num_splits));
    at::Tensor ws;
    if (workspace.has_value()) {
        ws = *workspace;
        require(ws.is_cuda() && ws.device() == q.device() && ws.is_contiguous() && ws.scalar_type() == at::kByte &&
                    size_t(ws.numel()) >= ws_bytes,
                "workspace must be a contiguous uint8 GPU tensor of at least paged_decode_workspace_bytes(...) bytes");
    } else {
        ws = at::empty({int64_t(ws_bytes)}, q.options().dtype(at::kByte));
    }
    const int st = fq_tq4_store_and_decode(
        kc.data_ptr(), vc.data_ptr(), sm.data_ptr<int64_t>(), re.data_ptr<float>(), ro.data_ptr<float>(),
        bd.data_ptr<float>(), qc.data_ptr(), kv_cache.data_ptr<uint8_t>(), bt.data_ptr<int32_t>(), sl.data_ptr<int32_t>(),
        ck.data_ptr<float>(), cv.data_ptr<float>(), rot.ptr, rot.col_major, result.data_ptr(), int(S), int(HQ), int(H),
        int(D), int(block_size), max_blocks, kv_cache.size(0), float(scale),
        fqbind::dtype_code(q.scalar_type(), "tq4_store_and_decode"), int(num_splits), ws.data_ptr(), size_t(ws.numel()),
        fqbind::current_stream(q));
    fqbind::raise_on_error(st, "tq4_store_and_decode");
    return result;
}

// Keys or values of (B, H, N, X) taken from a buffer of larger token capacity: a view
// buffer[:, :, :N, :] (the reference's CompressedBuffer.get(), src/flashquant/cache/buffer_pool.py:128-140)
// keeps the row layout of a contiguous tensor with N replaced by the capacity.  Returns that
// capacity, or 0 when the strides are anything else.
int64_t slab_capacity(const at::Tensor& t) {
    const int64_t B = t.size(0), H = t.size(1), N = t.size(2), X = t.size(3);
    if (t.numel() == 0) return N;
    if ((X > 1 && t.stride(3) != 1) || (N > 1 && t.stride(2) != X)) return 0;
    int64_t cap = N;
    if (H > 1) {
        if (t.stride(1) % X != 0) return 0;
        cap = t.stride(1) / X;
    } else if (B > 1) {
        if (t.stride(0) % X != 0) return 0;
        cap = t.stride(0) / X;
    }
    if (cap < N) return 0;
    if (B > 1 && t.stride(0) != H * cap * X) return 0;
    return cap;
}

// TQ4 compress of (B, H, n, D) new tokens straight into pre-allocated buffers at `position`:
// the compress + CompressedBuffer.append of the HF cache in one launch
// (src/flashquant/cache/hf_cache.py:283-312, src/flashquant/cache/buffer_pool.py:86-111).
void tq4_compress_append(const at::Tensor& x, const at::Tensor& rot_T_even, const at::Tensor& rot_T_odd,
                         const at::Tensor& boundaries, const at::Tensor& packed_buf, const at::Tensor& norms_buf,
                         int64_t position) {
    fqbind::require_gpu(x, "x");
    fqbind::require_gpu(packed_buf, "packed_buf");
    fqbind::require_gpu(norms_buf, "norms_buf");
    require(x.dim() == 4, "x must have shape (B, H, n, D)");
    require(x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16, "x must be float16 or bfloat16");
    const int64_t B = x.size(0), H = x.size(1), n = x.size(2), D = x.size(3);
    require(packed_buf.dim() == 4 && packed_buf.scalar_type() == at::kByte && packed_buf.is_contiguous() &&
                packed_buf.size(0) == B && packed_buf.size(1) == H && packed_buf.size(3) == D / 2,
            "packed_buf must be a contiguous uint8 buffer of shape (B, H, capacity, D/2)");
    const int64_t cap = packed_buf.size(2);
    require(norms_buf.scalar_type() == at::kFloat && norms_buf.is_contiguous() && norms_buf.numel() == B * H * cap,
            "norms_buf must be a contiguous float32 buffer of shape (B, H, capacity, 1)");
    if (position < 0 || position + n > cap)
        throw std::runtime_error("tq4_compress_append: appending " + std::to_string(n) + " tokens at position " +
                                 std::to_string(position) + " would exceed the capacity " + std::to_string(cap));
    require(rot_T_even.scalar_type() == at::kFloat && rot_T_odd.scalar_type() == at::kFloat &&
                boundaries.scalar_type() == at::kFloat && rot_T_even.dim() == 2 && rot_T_even.size(0) == D &&
                rot_T_even.size(1) == D / 2 && rot_T_odd.sizes() == rot_T_even.sizes() && boundaries.numel() == 15,
            "rotation halves must be float32 (D, D/2) and boundaries 15 float32 values");
    c10::DeviceGuard guard(x.device());
    const at::Tensor xc = x.contiguous();
    const at::Tensor re = rot_T_even.to(x.device()).contiguous(), ro = rot_T_odd.to(x.device()).contiguous();
    const at::Tensor bd = boundaries.to(x.device()).contiguous();
    const int st = fq_tq4_compress_append(xc.data_ptr(), fqbind::dtype_code(x.scalar_type(), "tq4_compress_append"),
                                          re.data_ptr<float>(), ro.data_ptr<float>(), bd.data_ptr<float>(),
                                          packed_buf.data_ptr<uint8_t>(), norms_buf.data_ptr<float>(), B * H, n, cap,
                                          position, int(D), fqbind::current_stream(x));
    fqbind::raise_on_error(st, "tq4_compress_append");
}

at::Tensor fused_tq_attention(const at::Tensor& q, const at::Tensor& k_packed, const at::Tensor& k_norms,
                              const at::Tensor& v_packed, const at::Tensor& v_norms, const at::Tensor& centroids_k,
                              const at::Tensor& centroids_v, const at::Tensor& rotation,
                              std::optional<double> sm_scale, bool is_causal) {
    fqbind::require_gpu(q, "q");
    fqbind::require_gpu(k_packed, "k_packed");
    fqbind::require_gpu(v_packed, "v_packed");
    require(q.dim() == 4, "q must have shape (B, H_Q, N_Q, D)");
    require(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "q must be float16 or bfloat16");
    const int64_t B = q.size(0), HQ = q.size(1), NQ = q.size(2), D = q.size(3);
    require(k_packed.dim() == 4 && k_packed.scalar_type() == at::kByte && k_packed.size(0) == B &&
                k_packed.size(3) == D / 2,
            "k_packed must be uint8 of shape (B, H_KV, N_KV, D/2)");
    const int64_t HKV = k_packed.size(1), NKV = k_packed.size(2);
    require(v_packed.scalar_type() == at::kByte && v_packed.sizes() == k_packed.sizes(),
            "v_packed must be uint8 with the shape of k_packed");
    require(HKV > 0 && HQ % HKV == 0, "H_Q must be a multiple of H_KV");
    require(k_norms.scalar_type() == at::kFloat && k_norms.numel() == B * HKV * NKV &&
                v_norms.scalar_type() == at::kFloat && v_norms.numel() == B * HKV * NKV,
            "norms must be float32 with one value per (batch, KV head, token)");
    require(centroids_k.numel() == 16 && centroids_v.numel() == 16 && centroids_k.scalar_type() == at::kFloat &&
                centroids_v.scalar_type() == at::kFloat,
            "centroids must be 16 float32 values");
    c10::DeviceGuard guard(q.device());
    const double scale = sm_scale.has_value() ? *sm_scale : 1.0 / std::sqrt(double(D));
    const at::Tensor qc = q.contiguous();
    // views of buffers with a larger token capacity are taken as they are (no copy)
    at::Tensor kp = k_packed, vp = v_packed;
    at::Tensor kn = k_norms.to(q.device()), vn = v_norms.to(q.device());
    if (kn.dim() != 4) kn = kn.reshape({B, HKV, NKV, 1});
    if (vn.dim() != 4) vn = vn.reshape({B, HKV, NKV, 1});
    int64_t k_cap = slab_capacity(kp), v_cap = slab_capacity(vp);
    if (k_cap == 0 || slab_capacity(kn) != k_cap) {
        kp = kp.contiguous();
        kn = kn.contiguous();
        k_cap = NKV;
    }
    if (v_cap == 0 || slab_capacity(vn) != v_cap) {
        vp = vp.contiguous();
        vn = vn.contiguous();
        v_cap = NKV;
    }
    const at::Tensor ck = centroids_k.to(q.device()).contiguous(), cv = centroids_v.to(q.device()).contiguous();
    const RotationArg rot = rotation_arg(rotation, q.device(), D);
    at::Tensor result = at::empty_like(qc);
    const int st = fq_fused_tq_attention_strided(
        qc.data_ptr(), kp.data_ptr<uint8_t>(), kn.data_ptr<float>(), vp.data_ptr<uint8_t>(), vn.data_ptr<float>(),
        ck.data_ptr<float>(), cv.data_ptr<float>(), rot.ptr, rot.col_major, result.data_ptr(),
        int(B), int(HQ), int(HKV), int(NQ), int(NKV), k_cap, v_cap, int(D), float(scale), is_causal ? 1 : 0,
        fqbind::dtype_code(q.scalar_type(), "fused_tq_attention"), fqbind::current_stream(q));
    fqbind::raise_on_error(st, "fused_tq_attention");
    return result;
}

at::Tensor paged_tq4_prefill(const at::Tensor& q, const at::Tensor& cu_seqlens_q, int64_t max_seqlen_q,
                             const at::Tensor& kv_cache, const at::Tensor& block_table, const at::Tensor& seq_lens,
                             const at::Tensor& centroids_k, const at::Tensor& centroids_v,
                             const at::Tensor& rotation, int64_t num_kv_heads, int64_t head_dim, int64_t block_size,
                             std::optional<double> sm_scale, bool causal, std::optional<at::Tensor> out) {
    fqbind::require_gpu(q, "q");
    fqbind::require_gpu(kv_cache, "kv_cache");
    fqbind::require_gpu(block_table, "block_table");
    fqbind::require_gpu(seq_lens, "seq_lens");
    fqbind::require_gpu(cu_seqlens_q, "cu_seqlens_q");
    require(q.dim() == 3 && q.size(2) == head_dim, "q must have shape (tokens, H_Q, head_dim)");
    require(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "q must be float16 or bfloat16");
    const int64_t T = q.size(0), HQ = q.size(1);
    require(num_kv_heads > 0 && HQ % num_kv_heads == 0, "H_Q must be a multiple of num_kv_heads");
    require(kv_cache.dim() == 3 && kv_cache.scalar_type() == at::kByte && kv_cache.size(1) == block_size &&
                kv_cache.size(2) == num_kv_heads * (head_dim + 8) && kv_cache.is_contiguous(),
            "kv_cache must be contiguous uint8 of shape (num_blocks, block_size, H_KV * (head_dim + 8))");
    require(block_table.dim() == 2 && block_table.scalar_type() == at::kInt, "block_table must be int32 (S, max_blocks)");
    const int64_t S = block_table.size(0);
    require(seq_lens.scalar_type() == at::kInt && seq_lens.numel() == S, "seq_lens must be int32 of shape (S,)");
    require(cu_seqlens_q.scalar_type() == at::kInt && cu_seqlens_q.numel() == S + 1,
            "cu_seqlens_q must be int32 of shape (S + 1,)");
    require(max_seqlen_q >= 0 && max_seqlen_q <= T, "max_seqlen_q must lie in [0, tokens]");
    require(centroids_k.numel() == 16 && centroids_v.numel() == 16 && centroids_k.scalar_type() == at::kFloat &&
                centroids_v.scalar_type() == at::kFloat,
            "centroids must be 16 float32 values");
    c10::DeviceGuard guard(q.device());
    const double scale = sm_scale.has_value() ? *sm_scale : 1.0 / std::sqrt(double(head_dim));
    const at::Tensor qc = q.contiguous();
    const at::Tensor bt = block_table.contiguous(), sl = seq_lens.contiguous(), cu = cu_seqlens_q.contiguous();
    const at::Tensor ck = centroids_k.to(q.device()).contiguous(), cv = centroids_v.to(q.device()).contiguous();
    const RotationArg rot = rotation_arg(rotation, q.device(), head_dim);
    at::Tensor result;
    if (out.has_value()) {
        require(out->sizes() == qc.sizes() && out->scalar_type() == q.scalar_type() && out->is_contiguous() &&
                    out->device() == q.device(),
                "out must be contiguous with the shape, dtype and device of q");
        result = *out;
    } else {
        result = at::zeros_like(qc);
    }
    const int st = fq_paged_tq4_prefill(
        qc.data_ptr(), cu.data_ptr<int32_t>(), kv_cache.data_ptr<uint8_t>(), bt.data_ptr<int32_t>(),
        sl.data_ptr<int32_t>(), ck.data_ptr<float>(), cv.data_ptr<float>(), rot.ptr, rot.col_major, result.data_ptr(),
        int(S), int(max_seqlen_q), int(HQ), int(num_kv_heads), int(head_dim), int(block_size), int(bt.size(1)),
        kv_cache.size(0), float(scale), causal ? 1 : 0, fqbind::dtype_code(q.scalar_type(), "paged_tq4_prefill"),
        fqbind::current_stream(q));
    fqbind::raise_on_error(st, "paged_tq4_prefill");
    return result;
}

std::tuple<at::Tensor, at::Tensor, at::Tensor> prod_compress(const at::Tensor& x, const at::Tensor& rotation,
                                                             const at::Tensor& sketch_rot, const at::Tensor& boundaries,
                                                             const at::Tensor& centroids) {
    fqbind::require_gpu(x, "x");
    require(x.dim() == 3, "x must have shape (N, H, D)");
    require(x.scalar_type() == at::kHalf || x.scalar_type() == at::kBFloat16, "x must be float16 or bfloat16");
    const int64_t N = x.size(0), H = x.size(1), D = x.size(2);
    require(boundaries.numel() == 7 && centroids.numel() == 8 && boundaries.scalar_type() == at::kFloat &&
                centroids.scalar_type() == at::kFloat,
            "the 3-bit codebook has 7 float32 boundaries and 8 float32 centroids");
    require(sketch_rot.dim() == 2 && sketch_rot.size(0) == D && sketch_rot.size(1) == D &&
                sketch_rot.scalar_type() == at::kFloat,
            "sketch_rot must be float32 of shape (D, D)");
    c10::DeviceGuard guard(x.device());
    const at::Tensor xc = x.contiguous();
    const RotationArg rot = rotation_arg(rotation, x.device(), D);
    const at::Tensor w = sketch_rot.to(x.device()).contiguous();
    const at::Tensor bd = boundaries.to(x.device()).contiguous(), ce = centroids.to(x.device()).contiguous();
    at::Tensor packed = at::empty({N, H, D / 2}, x.options().dtype(at::kByte));
    at::Tensor norms = at::empty({N, H, 1}, x.options().dtype(at::kFloat));
    at::Tensor gam = at::empty({N, H, 1}, x.options().dtype(at::kFloat));
    const int st = fq_prod_compress(xc.data_ptr(), fqbind::dtype_code(x.scalar_type(), "prod_compress"), rot.ptr,
                                    rot.col_major, w.data_ptr<float>(), bd.data_ptr<float>(), ce.data_ptr<float>(),
                                    packed.data_ptr<uint8_t>(), norms.data_ptr<float>(), gam.data_ptr<float>(), N * H,
                                    int(D), fqbind::current_stream(x));
    fqbind::raise_on_error(st, "prod_compress");
    return {packed, norms, gam};
}

at::Tensor prod_paged_decode(const at::Tensor& q, const at::Tensor& kv_cache, const at::Tensor& block_table,
                             const at::Tensor& seq_lens, const at::Tensor& centroids_k3, const at::Tensor& centroids_v,
                             const at::Tensor& rotation, const at::Tensor& sketch, int64_t num_kv_heads,
                             int64_t head_dim, int64_t block_size, std::optional<double> sm_scale,
                             const std::optional<at::Tensor>& out, int64_t num_splits) {
    fqbind::require_gpu(q, "q");
    fqbind::require_gpu(kv_cache, "kv_cache");
    require(q.dim() == 3 && q.size(2) == head_dim, "q must have shape (num_seqs, H_Q, D)");
    require(q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16, "q must be float16 or bfloat16");
    require(kv_cache.dim() == 3 && kv_cache.scalar_type() == at::kByte && kv_cache.is_contiguous() &&
                kv_cache.size(1) == block_size && kv_cache.size(2) == num_kv_heads * (head_dim + 12),
            "kv_cache must be contiguous uint8 of shape (num_blocks, block_size, num_kv_heads * (head_dim + 12))");
    require(block_table.dim() == 2 && block_table.scalar_type() == at::kInt && block_table.size(0) == q.size(0),
            "block_table must be int32 of shape (num_seqs, max_blocks)");
    require(seq_lens.scalar_type() == at::kInt && seq_lens.numel() == q.size(0), "seq_lens must be int32 (num_seqs,)");
    require(centroids_k3.numel() == 8 && centroids_v.numel() == 16 && centroids_k3.scalar_type() == at::kFloat &&
                centroids_v.scalar_type() == at::kFloat,
            "centroids_k3 must hold 8 and centroids_v 16 float32 values");
    require(sketch.dim() == 2 && sketch.size(0) == head_dim && sketch.size(1) == head_dim &&
                sketch.scalar_type() == at::kFloat,
            "sketch must be float32 of shape (D, D)");
    require(num_splits >= 0, "num_splits must be >= 0");
    c10::DeviceGuard guard(q.device());
    const int S = int(q.size(0)), HQ = int(q.size(1)), D = int(head_dim);
    const double scale = sm_scale.has_value() ? *sm_scale : 1.0 / std::sqrt(double(head_dim));
    const at::Tensor qc = q.contiguous();
    const at::Tensor bt = block_table.to(q.device()).contiguous();
    const at::Tensor sl = seq_lens.to(q.device()).contiguous();
    const at::Tensor ck = centroids_k3.to(q.device()).contiguous(), cv = centroids_v.to(q.device()).contiguous();
    const RotationArg rot = rotation_arg(rotation, q.device(), D);
    const at::Tensor sk = sketch.to(q.device()).contiguous();
    at::Tensor result;
    if (out.has_value()) {
        result = *out;
        require(result.is_cuda() && result.is_contiguous() && result.scalar_type() == q.scalar_type() &&
                    result.sizes() == q.sizes(),
                "out must be a contiguous GPU tensor with the shape and dtype of q");
    } else {
        result = at::empty_like(qc);
    }
    const int max_blocks = int(bt.size(1));
    const size_t ws_bytes = fq_paged_decode_workspace_bytes(S, HQ, int(num_kv_heads), D, int(block_size), max_blocks,
                                                            int(num_splits));
    at::Tensor ws = at::empty({int64_t(ws_bytes)}, q.options().dtype(at::kByte));
    const int st = fq_prod_paged_decode(
        qc.data_ptr(), kv_cache.data_ptr<uint8_t>(), bt.data_ptr<int32_t>(), sl.data_ptr<int32_t>(), ck.data_ptr<float>(),
        cv.data_ptr<float>(), rot.ptr, rot.col_major, sk.data_ptr<float>(), result.data_ptr(), S, HQ, int(num_kv_heads), D,
        int(block_size), max_blocks, kv_cache.size(0), float(scale), fqbind::dtype_code(q.scalar_type(), "prod_paged_decode"),
        int(num_splits), ws.data_ptr(), ws_bytes, fqbind::current_stream(q));
    fqbind::raise_on_error(st, "prod_paged_decode");
    return result;
}

at::Tensor nibble_pack(const at::Tensor& indices) {
    fqbind::require_gpu(indices, "indices");
    require(indices.dim() >= 1 && indices.size(-1) % 2 == 0, "Last dimension must be even for nibble packing");
    int bytes = 0;
    switch (indices.scalar_type()) {
        case at::kByte: bytes = 1; break;
        case at::kInt: bytes = 4; break;
        case at::kLong: bytes = 8; break;
        default: throw std::invalid_argument("nibble_pack: indices must be uint8, int32 or int64");
    }
    c10::DeviceGuard guard(indices.device());
    const at::Tensor ic = indices.contiguous();
    auto shape = ic.sizes().vec();
    shape.back() /= 2;
    at::Tensor packed = at::empty(shape, ic.options().dtype(at::kByte));
    at::Tensor bad = at::zeros({1}, ic.options().dtype(at::kInt));
    const int st = fq_nibble_pack(ic.data_ptr(), bytes, packed.data_ptr<uint8_t>(), packed.numel(), bad.data_ptr<int>(),
                                  fqbind::current_stream(indices));
    fqbind::raise_on_error(st, "nibble_pack");
    // the reference validates before it packs (csrc/core/packing.cpp:8-19): same error, after the fact
    if (bad.item<int>() != 0) throw std::invalid_argument("Indices out of range for 4-bit packing. Expected [0, 15]");
    return packed;
}

at::Tensor nibble_unpack(const at::Tensor& packed) {
    fqbind::require_gpu(packed, "packed");
    require(packed.scalar_type() == at::kByte, "nibble_unpack: packed must be uint8");
    c10::DeviceGuard guard(packed.device());
    const at::Tensor pc = packed.contiguous();
    auto shape = pc.sizes().vec();
    shape.back() *= 2;
    at::Tensor out = at::empty(shape, pc.options().dtype(at::kLong));
    const int st = fq_nibble_unpack(pc.data_ptr<uint8_t>(), out.data_ptr<int64_t>(), pc.numel(),
                                    fqbind::current_stream(packed));
    fqbind::raise_on_error(st, "nibble_unpack");
    return out;
}

at::Tensor pack_2bit(const at::Tensor& indices) {
    fqbind::require_gpu(indices, "indices");
    require(indices.dim() >= 1 && indices.size(-1) % 4 == 0, "Last dim must be divisible by 4");
    int bytes = 0;
    switch (indices.scalar_type()) {
        case at::kByte: bytes = 1; break;
        case at::kInt: bytes = 4; break;
        case at::kLong: bytes = 8; break;
        default: throw std::invalid_argument("pack_2bit: indices must be uint8, int32 or int64");
    }
    c10::DeviceGuard guard(indices.device());
    const at::Tensor ic = indices.contiguous();
    auto shape = ic.sizes().vec();
    shape.back() /= 4;
    at::Tensor packed = at::empty(shape, ic.options().dtype(at::kByte));
    at::Tensor bad = at::zeros({1}, ic.options().dtype(at::kInt));
    const int st = fq_pack_2bit(ic.data_ptr(), bytes, packed.data_ptr<uint8_t>(), packed.numel(), bad.data_ptr<int>(),
                                fqbind::current_stream(indices));
    fqbind::raise_on_error(st, "pack_2bit");
    if (bad.item<int>() != 0) throw std::invalid_argument("Indices out of range for 2-bit packing. Expected [0, 3]");
    return packed;
}

at::Tensor unpack_2bit(const at::Tensor& packed) {
    fqbind::require_gpu(packed, "packed");
    require(packed.scalar_type() == at::kByte, "unpack_2bit: packed must be uint8");
    c10::DeviceGuard guard(packed.device());
    const at::Tensor pc = packed.contiguous();
    auto shape = pc.sizes().vec();
    shape.back() *= 4;
    at::Tensor out = at::empty(shape, pc.options().dtype(at::kLong));
    const int st = fq_unpack_2bit(pc.data_ptr<uint8_t>(), out.data_ptr<int64_t>(), pc.numel(),
                                  fqbind::current_stream(packed));
    fqbind::raise_on_error(st, "unpack_2bit");
    return out;
}

// validate_indices (csrc/core/packing.cpp:8-19): raises when an index lies outside [0, 2^bits).
void validate_indices(const at::Tensor& indices, int64_t bits) {
    fqbind::require_gpu(indices, "indices");
    require(bits >= 1 && bits <= 8, "bits must lie in 1..8");
    if (indices.numel() == 0) return;
    const int64_t lo = indices.min().item<int64_t>(), hi = indices.max().item<int64_t>();
    if (lo < 0 || hi >= (int64_t(1) << bits))
        throw std::invalid_argument("Indices out of range for " + std::to_string(bits) + "-bit packing");
}

at::Tensor rotate_query(const at::Tensor& q, const at::Tensor& rotation) {
    fqbind::require_gpu(q, "q");
    require(q.dim() == 3 && (q.scalar_type() == at::kHalf || q.scalar_type() == at::kBFloat16),
            "q must be float16/bfloat16 of shape (num_seqs, H_Q, D)");
    c10::DeviceGuard guard(q.device());
    const at::Tensor qc = q.contiguous();
    const RotationArg rot = rotation_arg(rotation, q.device(), q.size(2));
    at::Tensor out = at::empty_like(qc);
    const int st = fq_rotate_query(qc.data_ptr(), rot.ptr, rot.col_major, out.data_ptr(), q.size(0), int(q.size(1)),
                                   int(q.size(2)), fqbind::dtype_code(q.scalar_type(), "rotate_query"),
                                   fqbind::current_stream(q));
    fqbind::raise_on_error(st, "rotate_query");
    return out;
}

using OptTriple = std::optional<std::tuple<at::Tensor, at::Tensor, at::Tensor>>;

std::tuple<at::Tensor, at::Tensor, at::Tensor> paged_tq4_decode_partials(
    const at::Tensor& q_rot, const at::Tensor& kv_cache, const at::Tensor& block_table, const at::Tensor& seq_lens,
    const at::Tensor& centroids_k, const at::Tensor& centroids_v, int64_t num_kv_heads, int64_t head_dim,
    int64_t block_size, double sm_scale, int64_t num_splits, const OptTriple& out,
    const std::optional<at::Tensor>& rotation) {
    fqbind::require_gpu(q_rot, "q_rot");
    fqbind::require_gpu(kv_cache, "kv_cache");
    require(q_rot.dim() == 3 && q_rot.size(2) == head_dim && q_rot.is_contiguous(), "q_rot must be contiguous (S, H_Q, D)");
    require(kv_cache.dim() == 3 && kv_cache.scalar_type() == at::kByte && kv_cache.is_contiguous() &&
                kv_cache.size(1) == block_size && kv_cache.size(2) == num_kv_heads * (head_dim + 8),
            "kv_cache must be contiguous uint8 (num_blocks, block_size, num_kv_heads * (head_dim + 8))");
    require(block_table.is_cuda() && block_table.is_contiguous() && block_table.scalar_type() == at::kInt &&
                block_table.dim() == 2 && block_table.size(0) == q_rot.size(0),
            "block_table must be a contiguous int32 GPU tensor (S, max_blocks)");
    require(seq_lens.is_cuda() && seq_lens.is_contiguous() && seq_lens.scalar_type() == at::kInt &&
                seq_lens.numel() == q_rot.size(0),
            "seq_lens must be a contiguous int32 GPU tensor (S,)");
    require(centroids_k.is_cuda() && centroids_v.is_cuda() && centroids_k.numel() == 16 && centroids_v.numel() == 16 &&
                centroids_k.scalar_type() == at::kFloat && centroids_v.scalar_type() == at::kFloat,
            "centroids must be 16 float32 values on the GPU");
    require(num_splits >= 1, "num_splits must be >= 1");
    c10::DeviceGuard guard(q_rot.device());
    const int64_t S = q_rot.size(0), HQ = q_rot.size(1);
    at::Tensor acc, m, l;
    if (out.has_value()) {
        acc = std::get<0>(*out); m = std::get<1>(*out); l = std::get<2>(*out);
        require(acc.is_cuda() && acc.is_contiguous() && acc.scalar_type() == at::kFloat &&
                    acc.numel() == S * HQ * num_splits * head_dim && m.is_cuda() && m.is_contiguous() &&
                    m.scalar_type() == at::kFloat && m.numel() == S * HQ * num_splits && l.is_cuda() &&
                    l.is_contiguous() && l.scalar_type() == at::kFloat && l.numel() == S * HQ * num_splits,
                "out must be float32 GPU tensors (S, H_Q, splits, D), (S, H_Q, splits), (S, H_Q, splits)");
    } else {
        acc = at::empty({S, HQ, num_splits, head_dim}, q_rot.options().dtype(at::kFloat));
        m = at::empty({S, HQ, num_splits}, q_rot.options().dtype(at::kFloat));
        l = at::empty({S, HQ, num_splits}, q_rot.options().dtype(at::kFloat));
    }
    RotationArg rot;
    if (rotation.has_value()) rot = rotation_arg(*rotation, q_rot.device(), head_dim);
    const int st = fq_paged_tq4_decode(
        q_rot.data_ptr(), rot.ptr, rot.col_major, kv_cache.data_ptr<uint8_t>(), block_table.data_ptr<int32_t>(), seq_lens.data_ptr<int32_t>(),
        centroids_k.data_ptr<float>(), centroids_v.data_ptr<float>(), acc.data_ptr<float>(), m.data_ptr<float>(),
        l.data_ptr<float>(), int(S), int(HQ), int(num_kv_heads), int(head_dim), int(block_size),
        int(block_table.size(1)), kv_cache.size(0), float(sm_scale),
        fqbind::dtype_code(q_rot.scalar_type(), "paged_tq4_decode_partials"), int(num_splits),
        fqbind::current_stream(q_rot));
    fqbind::raise_on_error(st, "paged_tq4_decode_partials");
    return {acc, m, l};
}

at::Tensor split_k_reduce(const at::Tensor& acc, const at::Tensor& m, const at::Tensor& l,
                          const std::optional<at::Tensor>& rotation, at::ScalarType dtype) {
    fqbind::require_gpu(acc, "partial_acc");
    require(acc.dim() == 4 && acc.is_contiguous() && acc.scalar_type() == at::kFloat && m.is_contiguous() &&
                l.is_contiguous() && m.is_cuda() && l.is_cuda() && m.scalar_type() == at::kFloat &&
                l.scalar_type() == at::kFloat && m.numel() == acc.numel() / acc.size(3) && l.numel() == m.numel(),
            "partials must be contiguous float32 GPU tensors (S, H_Q, splits, D), (S, H_Q, splits) x2");
    c10::DeviceGuard guard(acc.device());
    RotationArg rot;
    if (rotation.has_value()) rot = rotation_arg(*rotation, acc.device(), acc.size(3));
    at::Tensor out = at::empty({acc.size(0), acc.size(1), acc.size(3)}, acc.options().dtype(dtype));
    const int st = fq_split_k_reduce(acc.data_ptr<float>(), m.data_ptr<float>(), l.data_ptr<float>(),
                                     rot.ptr, rot.col_major, out.data_ptr(), int(acc.size(0)),
                                     int(acc.size(1)), int(acc.size(3)), fqbind::dtype_code(dtype, "split_k_reduce"),
                                     int(acc.size(2)), fqbind::current_stream(acc));
    fqbind::raise_on_error(st, "split_k_reduce");
    return out;
}

}  // namespace

void bind_kernels(py::module_& m) {
    m.def("tq4_compress", &tq4_compress, py::arg("x"), py::arg("rotation_T_even"), py::arg("rotation_T_odd"),
          py::arg("boundaries"), py::arg("out") = py::none(),
          "TQ4 compress of (N, H, D) fp16/bf16 rows -> (packed (N, H, D/2) uint8, norms (N, H, 1) float32).");
    m.def("tq4_compress_store", &tq4_compress_store, py::arg("key"), py::arg("value"), py::arg("rotation_T_even"),
          py::arg("rotation_T_odd"), py::arg("boundaries"), py::arg("kv_cache"), py::arg("slot_mapping"),
          "Compress key and value (N, H, D) and write them into the packed paged cache at slot_mapping");
    m.def("tq4_decompress", &tq4_decompress, py::arg("packed"), py::arg("norms"), py::arg("centroids"),
          py::arg("dtype"), py::arg("out") = py::none(),
          "TQ4 decompress to (N, H, D) in dtype, rotated space.");
    m.def("tq4_store_and_decode", &tq4_store_and_decode, py::arg("key"), py::arg("value"), py::arg("slot_mapping"),
          py::arg("rotation_T_even"), py::arg("rotation_T_odd"), py::arg("boundaries"), py::arg("q"), py::arg("kv_cache"),
          py::arg("block_table"), py::arg("seq_lens"), py::arg("centroids_k"), py::arg("centroids_v"), py::arg("rotation"),
          py::arg("num_kv_heads"), py::arg("head_dim"), py::arg("block_size"), py::arg("sm_scale") = py::none(),
          py::arg("out") = py::none(), py::arg("num_splits") = 0, py::arg("workspace") = py::none(),
          "One serving step: every sequence's new token compressed into its cache row, then the split-K paged decode.");
    m.def("split_k_paged_decode", &split_k_paged_decode, py::arg("q"), py::arg("kv_cache"), py::arg("block_table"),
          py::arg("seq_lens"), py::arg("centroids_k"), py::arg("centroids_v"), py::arg("rotation"),
          py::arg("num_kv_heads"), py::arg("head_dim"), py::arg("block_size"), py::arg("sm_scale") = py::none(),
          py::arg("out") = py::none(), py::arg("num_splits") = 0, py::arg("workspace") = py::none(),
          "Split-K paged decode from the packed TQ4 cache; q un-rotated, result in the original space.  "
          "`workspace`: optional uint8 GPU scratch of paged_decode_workspace_bytes(...) bytes, contents arbitrary.");
    // Same operator under the name the vLLM attention impl looks for
    // (src/flashquant/vllm/impl.py:57-59, called with sm_scale= and out= keywords).
    m.def("split_k_paged_decode_static", &split_k_paged_decode_static, py::arg("q"), py::arg("kv_cache"),
          py::arg("block_table"), py::arg("seq_lens"), py::arg("centroids_k"), py::arg("centroids_v"),
          py::arg("rotation"), py::arg("num_kv_heads"), py::arg("head_dim"), py::arg("block_size"),
          py::arg("sm_scale"), py::arg("out"), py::arg("num_splits") = 0,
          "split_k_paged_decode on the library's static scratch array: allocates nothing (every tensor must "
          "already be on the GPU, contiguous, and `out` is required).");
    m.def("static_scratch_bytes", &fq_static_scratch_bytes);
    m.def("paged_decode_workspace_bytes", &fq_paged_decode_workspace_bytes, py::arg("num_seqs"), py::arg("num_q_heads"),
          py::arg("num_kv_heads"), py::arg("head_dim"), py::arg("block_size"), py::arg("max_blocks_per_seq"),
          py::arg("num_splits") = 0);
    m.def("fused_paged_tq4_decode", &split_k_paged_decode, py::arg("q"), py::arg("kv_cache"), py::arg("block_table"),
          py::arg("seq_lens"), py::arg("centroids_k"), py::arg("centroids_v"), py::arg("rotation"),
          py::arg("num_kv_heads"), py::arg("head_dim"), py::arg("block_size"), py::arg("sm_scale") = py::none(),
          py::arg("out") = py::none(), py::arg("num_splits") = 0, py::arg("workspace") = py::none(),
          "Alias of split_k_paged_decode.");
    m.def("fused_tq_attention", &fused_tq_attention, py::arg("q"), py::arg("k_packed"), py::arg("k_norms"),
          py::arg("v_packed"), py::arg("v_norms"), py::arg("centroids_k"), py::arg("centroids_v"), py::arg("rotation"),
          py::arg("sm_scale") = py::none(), py::arg("is_causal") = false,
          "Fused TQ4 attention: un-rotated q (B, H_Q, N_Q, D) over packed K/V, original-space output");
    m.def("paged_tq4_prefill", &paged_tq4_prefill, py::arg("q"), py::arg("cu_seqlens_q"), py::arg("max_seqlen_q"),
          py::arg("kv_cache"), py::arg("block_table"), py::arg("seq_lens"), py::arg("centroids_k"),
          py::arg("centroids_v"), py::arg("rotation"), py::arg("num_kv_heads"), py::arg("head_dim"),
          py::arg("block_size"), py::arg("sm_scale") = py::none(), py::arg("causal") = true,
          py::arg("out") = py::none(),
          "Variable-length prefill over the packed paged TQ4 cache: un-rotated q (tokens, H_Q, D), original-space output");
    m.def("prod_compress", &prod_compress, py::arg("x"), py::arg("rotation"), py::arg("sketch_rot"),
          py::arg("boundaries"), py::arg("centroids"),
          "TurboQuantProd key compress: (packed nibbles sign<<3|idx (N,H,D/2), norms (N,H,1), residual norms (N,H,1))");
    m.def("prod_paged_decode", &prod_paged_decode, py::arg("q"), py::arg("kv_cache"), py::arg("block_table"),
          py::arg("seq_lens"), py::arg("centroids_k3"), py::arg("centroids_v"), py::arg("rotation"), py::arg("sketch"),
          py::arg("num_kv_heads"), py::arg("head_dim"), py::arg("block_size"), py::arg("sm_scale") = py::none(),
          py::arg("out") = py::none(), py::arg("num_splits") = 0,
          "Split-K paged decode over TurboQuantProd key / TQ4 value pages");
    // nibble_pack / nibble_unpack live in the sub-module only: as top-level names the reference's
    // packing functions would call them with CPU tensors and no device test
    // (src/flashquant/core/packing.py:37, 75, 94), and these are GPU kernels.
    {
        py::module_ pk = m.def_submodule("packing", "Index packing on the GPU");
        pk.def("nibble_pack", &nibble_pack, py::arg("indices"));
        pk.def("nibble_unpack", &nibble_unpack, py::arg("packed"));
        pk.def("pack_2bit", &pack_2bit, py::arg("indices"), "Four 2-bit indices per byte, the first in the top bits");
        pk.def("unpack_2bit", &unpack_2bit, py::arg("packed"), "Inverse of pack_2bit, int64");
        pk.def("validate_indices", &validate_indices, py::arg("indices"), py::arg("bits"));
    }
    m.def("tq4_compress_append", &tq4_compress_append, py::arg("x"), py::arg("rot_T_even"), py::arg("rot_T_odd"),
          py::arg("boundaries"), py::arg("packed_buf"), py::arg("norms_buf"), py::arg("position"),
          "TQ4 compress of x (B, H, n, D) into packed_buf (B, H, capacity, D/2) / norms_buf (B, H, capacity, 1) at "
          "token `position`, in place");
    m.def("tq4_decompress_rotated", &tq4_decompress_rotated, py::arg("packed"), py::arg("norms"), py::arg("centroids"),
          py::arg("rotation"), py::arg("dtype"), py::arg("out") = py::none(),
          "tq4_decompress to dtype, then (x.float() @ rotation).to(dtype): original-space rows in one launch");
    m.def("set_option", [](const std::string& name, int value) {
              const int id = option_id(name);
              const int before = fq_get_option(id);
              fqbind::raise_on_error(fq_set_option(id, value), "set_option");
              return before;
          }, py::arg("name"), py::arg("value"),
          "Set a kernel-variant switch ('decode_copy_waves', 'decode_direct', 'decode_ring', 'attention_any_dim', "
          "'compress_three_terms': 0 / 1; 'reduce_rows': 0, 4, 8 or 16); returns the old value");
    m.def("get_option", [](const std::string& name) { return fq_get_option(option_id(name)); }, py::arg("name"));
    m.def("paged_decode_fault_count", []() {
              unsigned int n = 0;
              fqbind::raise_on_error(fq_paged_decode_fault_count(&n), "paged_decode_fault_count");
              return n;
          }, "Timed-out wavefront hand-offs of the staged decode kernel on the current device (synchronises)");
    m.def("rotate_query", &rotate_query, py::arg("q"), py::arg("rotation"),
          "q_rot = (q @ rotation.T) rounded to q's dtype.");
    m.def("paged_tq4_decode_partials", &paged_tq4_decode_partials, py::arg("q_rot"), py::arg("kv_cache"),
          py::arg("block_table"), py::arg("seq_lens"), py::arg("centroids_k"), py::arg("centroids_v"),
          py::arg("num_kv_heads"), py::arg("head_dim"), py::arg("block_size"), py::arg("sm_scale"),
          py::arg("num_splits"), py::arg("out") = py::none(), py::arg("rotation") = py::none(),
          "Split partials (acc, m, l) of the paged decode; the query is pre-rotated unless `rotation` is given "
          "(accepted only where the kernel rotates the query itself).");
    m.def("paged_decode_fuses_rotation", &fq_paged_decode_fuses_rotation, py::arg("head_dim"),
          py::arg("num_kv_heads"), py::arg("shared_codebook"));
    m.def("split_k_reduce", &split_k_reduce, py::arg("partial_acc"), py::arg("partial_m"), py::arg("partial_l"),
          py::arg("rotation"), py::arg("dtype"), "Log-sum-exp combine of split partials, optional post-rotation.");
    m.def("paged_decode_auto_splits", &fq_paged_decode_auto_splits, py::arg("num_seqs"), py::arg("num_kv_heads"),
          py::arg("block_size"), py::arg("max_blocks_per_seq"));
}
