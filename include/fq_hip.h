/*
 * fq_hip.h - C ABI of libfq_hip.so, the MI355X (gfx950) implementation of the
 * TurboQuant TQ4 KV-cache kernels.
 *
 * Every entry point takes plain device pointers, sizes and an opaque HIP
 * stream (hipStream_t passed as void*; NULL is the default stream), launches
 * asynchronously on that stream, allocates nothing, never synchronises and
 * never aborts: it returns an fq_status code.  All buffers are owned by the
 * caller.  Entry points whose kernels need scratch memory take a caller-owned
 * workspace whose size comes from the matching *_workspace_bytes() function.
 *
 * Each declaration cites the launcher of the reference (paths relative to the
 * reference checkout) whose role it takes, or the Python call site that
 * defines the operator where the reference has no working launcher.
 */
#ifndef FQ_HIP_H
#define FQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FQ_ABI_VERSION 1

typedef enum fq_status {
    FQ_OK = 0,
    FQ_ERR_NULL_POINTER = 1,      /* a required pointer argument is NULL           */
    FQ_ERR_UNSUPPORTED_DIM = 2,   /* head_dim not in {64, 128, 256}                */
    FQ_ERR_UNSUPPORTED_BLOCK = 3, /* page size not in {8, 16, 32}                  */
    FQ_ERR_UNSUPPORTED_DTYPE = 4, /* dtype code not accepted by this entry point   */
    FQ_ERR_BAD_SHAPE = 5,         /* negative size, H_Q not a multiple of H_KV ... */
    FQ_ERR_MISALIGNED = 6,        /* a pointer or stride breaks the stated alignment */
    FQ_ERR_WORKSPACE = 7,         /* workspace missing or too small                */
    FQ_ERR_LAUNCH = 8             /* the HIP runtime refused the launch            */
} fq_status;

typedef enum fq_dtype {
    FQ_F16 = 0,
    FQ_BF16 = 1,
    FQ_F32 = 2
} fq_dtype;

/*
 * Kernel-variant switches, for tests and measurements.  Each takes its first value from an
 * environment variable that is read once per process; fq_set_option changes it afterwards
 * (value 0 or 1), fq_get_option reads it (-1 for an unknown option).  Every entry point reads the
 * switches once, when it is called, so one call never mixes two settings; fq_set_option itself is not
 * ordered against calls running on other host threads, so change a switch only while no other thread
 * is inside the library.
 */
typedef enum fq_option {
    FQ_OPT_DECODE_COPY_WAVES = 0, /* FQ_DECODE_COPY_WAVES, default 1: the staged decode kernel runs with
                                     wavefronts that only copy; 0: its computing wavefronts copy too     */
    FQ_OPT_DECODE_DIRECT = 1,     /* FQ_DECODE_DIRECT, default 0: 1 sends every shape to the direct
                                     decode kernel                                                      */
    FQ_OPT_ATTENTION_ANY_DIM = 2, /* FQ_ATTENTION_ANY_DIM, default 0: 1 sends head_dim 128 to the general
                                     attention kernel                                                   */
    FQ_OPT_DECODE_TINY_SPIN = 3,  /* default 0: 1 makes the bounded waits between the wavefronts of the staged
                                     decode kernel give up after two polls, to exercise the failure path
                                     (NaN rows, fault counter) without hanging anything                */
    FQ_OPT_COMPRESS_THREE_TERMS = 4, /* FQ_COMPRESS_THREE_TERMS, default 0: bf16 rows of head_dim 64 / 128 are
                                     rotated against the matrix as two bf16 terms (|error| <= 2^-18 per
                                     element: about 6 indices in a million differ from the float32 result);
                                     1: three terms, the float32 matrix exactly, at 3/2 of the matrix work */
    FQ_OPT_DECODE_RING = 5,       /* FQ_DECODE_RING, default 0: 1 sends groups of 8 KV heads of dimension 128 to the
                                     ring decode kernel (16 computing wavefronts, direct-to-LDS loads)
                                     instead of the staged kernel with copy wavefronts                    */
    FQ_OPT_REDUCE_ROWS = 6,       /* FQ_REDUCE_ROWS, default 0: rows per workgroup of the combine kernel chosen from
                                     the row count; 4, 8 or 16 forces that many                          */
    FQ_OPTION_COUNT = 7
} fq_option;
int fq_get_option(int option);
int fq_set_option(int option, int value);

/* Library identification and error text. */
int fq_abi_version(void);
const char* fq_status_string(int status);
/* Text of the last HIP runtime error seen by this thread ("" if none).  An entry point that launches asks
 * the runtime for its last error after the launch (hipGetLastError, which also clears it): an error that
 * an earlier HIP call of the same thread left behind is therefore reported, as FQ_ERR_LAUNCH, by the next
 * entry point called, whose own launch may have been fine; this text names the error either way. */
const char* fq_last_hip_error(void);

/*
 * Lloyd-Max codebook of a rotated unit vector's coordinates: N(0, 1/dim) truncated
 * to +-3.5 sigma, 2^bits levels.  Host code, no GPU work.  Follows the solver the
 * reference's Python layer defines the kernel inputs with
 * (_gaussian_centroids_boundaries, src/flashquant/core/codebook.py:58-140), not
 * the numerically different csrc/core/codebook.cpp:64-121.
 *   centroids   (2^bits,) float32 out, host memory
 *   boundaries  (2^bits - 1,) float32 out, host memory: midpoints of the centroids
 * bits in 1..8.
 */
int fq_lloyd_max_gaussian(int dim, int bits, float* centroids, float* boundaries);

/*
 * TurboQuantMSE.quantize / dequantize for any bit width up to 4
 * (src/flashquant/core/quantizer.py:125-195; C++ twin csrc/core/quantizer.cpp:24-72),
 * float32 arithmetic on the GPU.
 *
 * fq_mse_quantize:    n = ||x||, y = (x / (n + 1e-10)) R^T, idx = #{boundaries < y}
 *   x            (M, D) fp16 / bf16 / float32 rows, contiguous
 *   rotation     (D, D) float32, 16-byte aligned; rotation_col_major != 0 when the
 *                buffer holds the transpose (layout as in fq_split_k_paged_decode)
 *   boundaries   (num_boundaries,) float32 ascending, 1 <= num_boundaries <= 15
 *   indices      (M, D) int64 out;  norms (M,) float32 out
 * fq_mse_dequantize:  out = (centroids[idx] R) n
 *   indices      (M, D) int64, clamped to [0, num_centroids - 1]
 *   out          (M, D) float32, original space
 * fq_mse_residual:    residual = x - (centroids[idx] R) n,  residual_norms = ||residual||
 *                     (the first half of TurboQuantProd.quantize, quantizer.py:287-295)
 * fq_project_rows:    out = x M^T in float32, or sign(x M^T) with 0 -> +1 when
 *                     signs_only != 0 (the sketch of TurboQuantProd, quantizer.py:297-304
 *                     and 357-359); matrix (D, D) float32
 * D in {64, 128, 256}.  M == 0 is a no-op.
 */
int fq_mse_quantize(const void* x, int x_dtype, const float* rotation, int rotation_col_major,
                    const float* boundaries, int num_boundaries, int64_t* indices, float* norms,
                    int64_t M, int D, void* stream);
int fq_mse_dequantize(const int64_t* indices, const float* norms, const float* rotation,
                      int rotation_col_major, const float* centroids, int num_centroids, float* out,
                      int64_t M, int D, void* stream);
int fq_mse_residual(const void* x, int x_dtype, const int64_t* indices, const float* norms,
                    const float* rotation, int rotation_col_major, const float* centroids,
                    int num_centroids, float* residual, float* residual_norms, int64_t M, int D,
                    void* stream);
int fq_project_rows(const void* x, int x_dtype, const float* matrix, int matrix_col_major, int signs_only,
                    float* out, int64_t M, int D, void* stream);

/*
 * TQ4 compress.  Takes the role of tq4_compress_cuda
 * (csrc/cuda/compress.cuh:38-48); operator defined by compress_reference
 * (src/flashquant/kernels/cpu_reference.py:22-61).
 *
 *   x           (M, D) fp16 or bf16 rows, contiguous, 16-byte aligned
 *   rot_T_even  (D, D/2) float32 = rotation.T[:, 0::2], contiguous
 *   rot_T_odd   (D, D/2) float32 = rotation.T[:, 1::2], contiguous
 *   boundaries  (15,) float32, ascending
 *   packed      (M, D/2) uint8 out, 16-byte aligned: byte j = idx[2j]<<4 | idx[2j+1]
 *   norms       (M,) float32 out
 * D in {64, 128, 256}.  M == 0 is a no-op.
 *
 * Precision of the rotation (this entry point, fq_tq4_compress_append and fq_tq4_compress_store
 * alike).  fp16 rows, and bf16 rows of head_dim 256, are rotated against two fp16 terms of the
 * matrix (22 bits: the float32 product to within summation order).  bf16 rows of head_dim 64 / 128
 * are by default rotated against TWO bf16 terms of the matrix (16 bits): a rotated coordinate is
 * then off by up to 1e-6, and 5 to 7 indices in a million land in the neighbouring bucket of the
 * reference's float32 result (each such coordinate lies within 2e-6 of a boundary).  The switch
 * FQ_OPT_COMPRESS_THREE_TERMS (environment FQ_COMPRESS_THREE_TERMS=1) adds the third term: the
 * float32 matrix exactly, indices equal to the reference's wherever the coordinate is not within
 * float32 rounding of a boundary, at about 1.2 x the time.
 */
int fq_tq4_compress(const void* x, int x_dtype,
                    const float* rot_T_even, const float* rot_T_odd,
                    const float* boundaries,
                    uint8_t* packed, float* norms,
                    int64_t M, int D, void* stream);

/*
 * TQ4 compress straight into a pre-allocated (B, H, capacity, D/2) buffer at a token position:
 * the compress of the HF cache followed by CompressedBuffer.append
 * (src/flashquant/cache/hf_cache.py:283-312, src/flashquant/cache/buffer_pool.py:86-111) without
 * the intermediate tensors or the strided copy.
 *   x          (outer, n_new, D) fp16 / bf16, contiguous: outer = B * H slabs of n_new new tokens
 *   packed     (outer, capacity, D/2) uint8 buffer, norms (outer, capacity) float32 buffer;
 *              row (o, t) of x lands in row (o, position + t)
 * position >= 0 and position + n_new <= capacity, else FQ_ERR_BAD_SHAPE (the reference raises
 * on overflow, buffer_pool.py:100-107).  Rotation precision and its switch: as fq_tq4_compress
 * (two bf16 matrix terms by default for bf16 rows of head_dim 64 / 128).
 */
int fq_tq4_compress_append(const void* x, int x_dtype,
                           const float* rot_T_even, const float* rot_T_odd, const float* boundaries,
                           uint8_t* packed, float* norms,
                           int64_t outer, int64_t n_new, int64_t capacity, int64_t position,
                           int D, void* stream);

/*
 * Fused compress-and-store: compresses key and value rows and writes them straight
 * into the packed paged cache, one launch.  Takes the place of the two tq4_compress
 * calls, the row assembly and the advanced-index scatter of _compress_and_store
 * (src/flashquant/vllm/impl.py:220-263); cache row layout of
 * src/flashquant/vllm/impl.py:132-138.
 *
 *   key, value    (num_tokens, H_KV, D) fp16 or bf16, contiguous, 16-byte aligned
 *   kv_cache      (num_slots, H_KV*(D+8)) uint8 viewed flat over (block, position), 16-byte aligned
 *   slot_mapping  (num_mapped,) int64: flat slot of token i; tokens i >= num_mapped are
 *                 not stored (impl.py:259-261).  A negative or out-of-range slot is
 *                 skipped (the reference's index assignment would wrap a negative one).
 * Tokens that map to the same slot race, as they do in the reference.  Rotation precision and
 * its switch: as fq_tq4_compress (two bf16 matrix terms by default for bf16 rows of head_dim
 * 64 / 128).
 */
int fq_tq4_compress_store(const void* key, const void* value, int x_dtype,
                          const float* rot_T_even, const float* rot_T_odd, const float* boundaries,
                          uint8_t* kv_cache, const int64_t* slot_mapping,
                          int64_t num_tokens, int64_t num_mapped, int H_KV, int D,
                          int64_t num_slots, void* stream);

/*
 * TQ4 decompress.  Takes the role of tq4_decompress_cuda
 * (csrc/cuda/decompress.cuh:40-48); operator defined by decompress_reference
 * (src/flashquant/kernels/cpu_reference.py:64-94) followed by the cast of
 * src/flashquant/kernels/decompress.py:80-81.
 *
 *   packed     (M, D/2) uint8, 4-byte aligned
 *   norms      (M,) float32
 *   centroids  (16,) float32
 *   out        (M, D) fp16 / bf16 / float32, 16-byte aligned; rotated space,
 *              out[2j] from the high nibble of byte j, out[2j+1] from the low
 */
int fq_tq4_decompress(const uint8_t* packed, const float* norms,
                      const float* centroids,
                      void* out, int out_dtype,
                      int64_t M, int D, void* stream);

/*
 * TQ4 decompress followed by the inverse rotation, one launch: what the serving path does
 * when it materialises the cache (_decompress_cache with apply_rotation,
 * src/flashquant/vllm/impl.py:265-318: tq4_decompress to the compute dtype, then
 * (x.float() @ rotation).to(dtype), impl.py:309-316).
 *
 *   packed, norms, centroids   as for fq_tq4_decompress
 *   rotation   (D, D) float32, layout flag as in fq_split_k_paged_decode
 *   out        (M, D) fp16 / bf16, 16-byte aligned, original space:
 *              out = dtype(float32(dtype(centroid[idx] * norm)) @ rotation)
 * The contraction accumulates in float32 on the matrix cores in an order of its own, so a
 * result may differ from a float32 matmul's by one unit in the last place of the 16-bit output.
 */
int fq_tq4_decompress_rotated(const uint8_t* packed, const float* norms, const float* centroids,
                              const float* rotation, int rotation_col_major,
                              void* out, int out_dtype, int64_t M, int D, void* stream);

/*
 * Fused TQ4 attention (prefill): un-rotated query, packed keys and values,
 * original-space output.  Takes the role of the reference's fused launcher
 * (csrc/cuda/fused_tq_attention.cu:468-479); operator defined by
 * fused_tq_attention_reference (src/flashquant/kernels/cpu_reference.py:154-227)
 * with the query pre-rotation of src/flashquant/kernels/attention.py:85-107.
 *
 *   q          (B, H_Q, N_Q, D) fp16/bf16, contiguous, 16-byte aligned
 *   k_packed   (B, H_KV, N_KV, D/2) uint8, contiguous; v_packed the same
 *   k_norms    (B, H_KV, N_KV) float32; v_norms the same
 *   centroids_k, centroids_v  (16,) float32
 *   rotation   (D, D) float32, layout as in fq_split_k_paged_decode
 *   out        (B, H_Q, N_Q, D) same dtype as q
 *   is_causal  key j > query i (counted from the top-left corner) is hidden;
 *              ignored when N_Q == 1, as in the reference
 * D in {64, 128, 256}: 128 runs the tuned kernel, 64 and 256 a general one
 * (the switch FQ_OPT_ATTENTION_ANY_DIM sends 128 there too).  H_Q a multiple
 * of H_KV; 1 <= N_KV <= 2^24.  K and V are dequantised to fp16 with the norm folded in, so a
 * row norm times a centroid must stay below 65504.
 */
int fq_fused_tq_attention(const void* q, const uint8_t* k_packed, const float* k_norms,
                          const uint8_t* v_packed, const float* v_norms,
                          const float* centroids_k, const float* centroids_v,
                          const float* rotation, int rotation_col_major, void* out,
                          int B, int H_Q, int H_KV, int N_Q, int N_KV, int D,
                          float sm_scale, int is_causal, int dtype, void* stream);

/*
 * The same with keys and values in pre-allocated buffers of a larger capacity: the views that
 * the reference's ring buffer hands out, CompressedBuffer.get()
 * (src/flashquant/cache/buffer_pool.py:128-140: indices[:, :, :len, :] of a (B, H, max_seq, D/2)
 * buffer, norms likewise), go in without a copy (the fused mode of the HF cache,
 * src/flashquant/cache/hf_cache.py:322-329, 387-414).
 *   k_capacity, v_capacity   tokens between the slabs of consecutive (batch, KV head) pairs in
 *                            the key and the value buffers (max_seq there), each >= N_KV
 */
int fq_fused_tq_attention_strided(const void* q, const uint8_t* k_packed, const float* k_norms,
                                  const uint8_t* v_packed, const float* v_norms,
                                  const float* centroids_k, const float* centroids_v,
                                  const float* rotation, int rotation_col_major, void* out,
                                  int B, int H_Q, int H_KV, int N_Q, int N_KV,
                                  int64_t k_capacity, int64_t v_capacity, int D,
                                  float sm_scale, int is_causal, int dtype, void* stream);

/*
 * Prefill over the packed paged TQ4 cache: un-rotated queries of several
 * sequences packed along the token axis, keys and values read from the cache
 * through the block table, original-space output.  One launch for what the
 * serving backend does in four steps: rotate the query, decompress the whole
 * cache to fp16/bf16, variable-length attention through the block table,
 * rotate the result back (src/flashquant/vllm/impl.py:317-336 and 470-512;
 * the decompression is impl.py:265-315).  The tokens' own keys and values must
 * already be in the cache (fq_tq4_compress_store), as in the reference, which
 * stores before it attends (impl.py:320-323).
 *
 *   q             (total_q, H_Q, D) fp16/bf16, contiguous, 16-byte aligned
 *   cu_seqlens_q  (num_seqs + 1,) int32, first query token of every sequence,
 *                 non-decreasing, cu_seqlens_q[num_seqs] == total_q
 *   kv_cache, block_table, seq_lens   as in fq_split_k_paged_decode; seq_lens
 *                 counts the new tokens too, so seq_lens[s] >= the sequence's
 *                 query count
 *   out           (total_q, H_Q, D) same dtype as q
 *   max_q_len     the largest query count of a sequence (sizes the grid)
 *   is_causal     query j of n in a sequence of L keys sees keys 0 .. L - n + j
 * The attention result is rounded to the query dtype before the rotation back,
 * as the attention library's output is in the reference.  A sequence with no
 * queries is skipped; with no keys its rows are zero.  D in {64, 128, 256} as for
 * fq_fused_tq_attention.
 */
int fq_paged_tq4_prefill(const void* q, const int32_t* cu_seqlens_q, const uint8_t* kv_cache,
                         const int32_t* block_table, const int32_t* seq_lens,
                         const float* centroids_k, const float* centroids_v,
                         const float* rotation, int rotation_col_major, void* out,
                         int num_seqs, int max_q_len, int H_Q, int H_KV, int D, int block_size,
                         int max_blocks_per_seq, int64_t num_blocks, float sm_scale, int is_causal,
                         int dtype, void* stream);

/*
 * Split-K paged decode from the packed TQ4 cache, un-rotated query in,
 * original-space output out.  Takes the roles of paged_tq4_decode_cuda
 * (csrc/cuda/paged_decode.cu:346-368) and split_k_reduce_cuda
 * (csrc/cuda/split_k_reduce.cu:145-154) together with the query pre-rotation
 * and output post-rotation of src/flashquant/kernels/paged_decode.py:112-128;
 * operator defined by paged_decode_reference
 * (src/flashquant/kernels/cpu_reference.py:230-368).
 *
 *   q            (S, H_Q, D) fp16/bf16, contiguous
 *   kv_cache     (num_blocks, block_size, H_KV*(D+8)) uint8, 16-byte aligned
 *   block_table  (S, max_blocks_per_seq) int32
 *   seq_lens     (S,) int32; a length of 0 gives a zero output row
 *   centroids_k, centroids_v  (16,) float32
 *   rotation     (D, D) float32, or NULL: q is taken as already rotated and
 *                out is left in rotated space
 *   rotation_col_major  0: element (i, j) at i*D + j; 1: at i + j*D (the layout
 *                of a LAPACK QR factor, whose transpose is the contiguous one)
 *   out          (S, H_Q, D) same dtype as q
 *   num_splits   >= 1, or 0 to let the library choose
 *   workspace    fq_paged_decode_workspace_bytes(...) bytes, 256-byte aligned
 * D in {64, 128, 256}; block_size in {8, 16, 32}; H_Q a multiple of H_KV with
 * H_Q / H_KV <= 16.
 */
int fq_split_k_paged_decode(const void* q, const uint8_t* kv_cache,
                            const int32_t* block_table, const int32_t* seq_lens,
                            const float* centroids_k, const float* centroids_v,
                            const float* rotation, int rotation_col_major, void* out,
                            int num_seqs, int H_Q, int H_KV, int D,
                            int block_size, int max_blocks_per_seq,
                            int64_t num_blocks, float sm_scale, int dtype,
                            int num_splits,
                            void* workspace, size_t workspace_bytes,
                            void* stream);

/*
 * One serving step in one call: the step's new token of every sequence is
 * compressed into its cache row (fq_tq4_compress_store on one token per
 * sequence), then the decode runs over the cache that holds it
 * (fq_split_k_paged_decode).  It is the sequence of
 * src/flashquant/vllm/impl.py:362-394 (_compress_and_store, then the decode
 * kernel) for a batch of single-token queries.
 *
 *   key, value    (S, H_KV, D) fp16/bf16 as q, contiguous, 16-byte aligned
 *   slot_mapping  (S,) int64: flat slot of sequence s's new token; negative or
 *                 out of range: not stored
 *   rot_T_even, rot_T_odd, boundaries   as for fq_tq4_compress_store
 *   kv_cache      read and written
 *   everything else as for fq_split_k_paged_decode; rotation must not be NULL;
 *   seq_lens counts the new token.
 * Where the staged decode kernel runs (D == 128 and H_KV a multiple of 8, or
 * H_KV == 1, 2 or 4 on pages of 16 or 32 tokens; D == 64 and H_KV == 2, 4 or 8 on
 * such pages, up to 8 query heads per KV head; default switches) this is one launch
 * fewer: the workgroup whose split ends with a
 * sequence's last token compresses and stores that token in its prologue and
 * reads the row back with its last tile.  For that form slot_mapping[s] must be
 * the slot of token seq_lens[s] - 1 of sequence s as the block table gives it
 * (block_table[s][(L-1) / block_size] * block_size + (L-1) % block_size), which
 * is what a decode step passes; a sequence of length 0 stores nothing.  The
 * rotation there is the exact float32 one (three bf16 terms), so the stored
 * indices are those of FQ_OPT_COMPRESS_THREE_TERMS.  Other shapes run the two
 * entry points one after the other.
 */
int fq_tq4_store_and_decode(const void* key, const void* value, const int64_t* slot_mapping,
                            const float* rot_T_even, const float* rot_T_odd, const float* boundaries,
                            const void* q, uint8_t* kv_cache, const int32_t* block_table,
                            const int32_t* seq_lens, const float* centroids_k, const float* centroids_v,
                            const float* rotation, int rotation_col_major, void* out, int num_seqs,
                            int H_Q, int H_KV, int D, int block_size, int max_blocks_per_seq,
                            int64_t num_blocks, float sm_scale, int dtype, int num_splits,
                            void* workspace, size_t workspace_bytes, void* stream);

/*
 * The three stages of fq_split_k_paged_decode as separate launches, for callers
 * that hold the rotated query or want the partials (the reference exposes its
 * decode at this level: paged_tq4_decode_cuda, csrc/cuda/paged_decode.cu:346-368,
 * and split_k_reduce_cuda, csrc/cuda/split_k_reduce.cu:145-154).
 *
 * fq_rotate_query:     q_rot = (q @ rotation.T) rounded to dtype
 *                      (src/flashquant/kernels/paged_decode.py:113); q, q_rot (num_seqs, H_Q, D).
 * fq_paged_tq4_decode: q pre-rotated and rotation NULL, or q un-rotated with the rotation,
 *                      which the kernel then applies itself: allowed only where
 *                      fq_paged_decode_fuses_rotation() returns 1 (8 KV heads of dimension
 *                      128), FQ_ERR_BAD_SHAPE elsewhere.
 *                      Writes un-normalised float32 partials
 *                      partial_acc (num_seqs, H_Q, num_splits, D) and the base-2 running
 *                      maximum / denominator partial_m, partial_l (num_seqs, H_Q, num_splits);
 *                      an empty split has m = -inf.  num_splits >= 1.
 * fq_split_k_reduce:   out = sum_s acc_s 2^(m_s - m*) / sum_s l_s 2^(m_s - m*), rounded to
 *                      dtype; if rotation is not NULL the rounded value is multiplied by
 *                      rotation in float32 and rounded again (paged_decode.py:123).
 */
int fq_rotate_query(const void* q, const float* rotation, int rotation_col_major, void* q_rot,
                    int64_t num_seqs, int H_Q, int D, int dtype, void* stream);

int fq_paged_decode_fuses_rotation(int D, int H_KV, int shared_codebook);

int fq_paged_tq4_decode(const void* q, const float* rotation, int rotation_col_major,
                        const uint8_t* kv_cache,
                        const int32_t* block_table, const int32_t* seq_lens,
                        const float* centroids_k, const float* centroids_v,
                        float* partial_acc, float* partial_m, float* partial_l,
                        int num_seqs, int H_Q, int H_KV, int D,
                        int block_size, int max_blocks_per_seq, int64_t num_blocks,
                        float sm_scale, int dtype, int num_splits, void* stream);

int fq_split_k_reduce(const float* partial_acc, const float* partial_m,
                      const float* partial_l, const float* rotation,
                      int rotation_col_major, void* out,
                      int num_seqs, int H_Q, int D, int dtype, int num_splits,
                      void* stream);

/*
 * Nibble pack / unpack of 4-bit indices (src/flashquant/core/packing.py:54-98; C++ twin
 * csrc/core/packing.cpp:21-46).
 *   fq_nibble_pack    indices: 2 * n_packed values of index_bytes (1: uint8, 4: int32, 8: int64)
 *                     bytes each; packed[j] = idx[2j] << 4 | idx[2j+1].  *bad_count (device int,
 *                     zeroed by the caller) is raised when an index lies outside [0, 15]: the
 *                     reference rejects such input (validate_indices, csrc/core/packing.cpp:8-19).
 *   fq_nibble_unpack  indices (int64, as the Python fallback returns): [high, low] interleaved.
 */
int fq_nibble_pack(const void* indices, int index_bytes, uint8_t* packed, int64_t n_packed,
                   int* bad_count, void* stream);
int fq_nibble_unpack(const uint8_t* packed, int64_t* indices, int64_t n_packed, void* stream);

/*
 * 2-bit packing, four indices per byte with the first in the top bits
 * (pack_2bit / unpack_2bit, csrc/core/packing.cpp:48-79).  Arguments as for the
 * nibble pair; n_packed = number of bytes; indices outside [0, 3] are counted in
 * *bad_count.
 */
int fq_pack_2bit(const void* indices, int index_bytes, uint8_t* packed, int64_t n_packed,
                 int* bad_count, void* stream);
int fq_unpack_2bit(const uint8_t* packed, int64_t* indices, int64_t n_packed, void* stream);

/*
 * TurboQuantProd keys (3-bit Lloyd-Max index + 1-bit sign sketch of the residual) with
 * TQ4 values, as pages.  The reference defines the quantizer
 * (TurboQuantProd.quantize / estimate_inner_product, src/flashquant/core/quantizer.py:285-370;
 * C++ twin csrc/core/quantizer.cpp:76-184) but has no paged or fused path for it, so the
 * packed record is this library's own:
 *
 *   key nibble   = sign_bit << 3 | index (sign_bit 1 where resid . S_j < 0), two per byte,
 *                  even coordinate in the high nibble
 *   token row    = [K nibbles H*D/2 | K norm H*4 | K residual norm H*4 | V idx H*D/2 | V norm H*4],
 *                  H*(D+12) bytes, norms little-endian float32
 *
 * fq_prod_compress: x (M, D) fp16/bf16 -> packed (M, D/2) uint8, norms (M,), residual_norms (M,).
 *   rotation    (D, D) float32 R, layout flag as in fq_split_k_paged_decode
 *   sketch_rot  (D, D) float32 row-major, S @ R.T for the (D, D) sketch S (computed once by the caller)
 *   boundaries  (7,), centroids (8,) float32: the 3-bit codebook
 * fq_prod_paged_decode: split-K decode over such pages, un-rotated query in, original-space
 *   output out: score = <q, k_mse> + gamma sqrt(pi/2)/D <S q, signs> (quantizer.py:355-370),
 *   softmax, TQ4 values.  sketch is S itself, (D, D) row-major.  Workspace and num_splits as in
 *   fq_split_k_paged_decode.  D == 128, H_KV a multiple of 8, H_Q / H_KV <= 8.
 */
int fq_prod_compress(const void* x, int x_dtype, const float* rotation, int rotation_col_major,
                     const float* sketch_rot, const float* boundaries, const float* centroids,
                     uint8_t* packed, float* norms, float* residual_norms, int64_t M, int D, void* stream);

int fq_prod_paged_decode(const void* q, const uint8_t* kv_cache, const int32_t* block_table,
                         const int32_t* seq_lens, const float* centroids_k3, const float* centroids_v,
                         const float* rotation, int rotation_col_major, const float* sketch, void* out,
                         int num_seqs, int H_Q, int H_KV, int D, int block_size, int max_blocks_per_seq,
                         int64_t num_blocks, float sm_scale, int dtype, int num_splits,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * The prologue of the staged decode kernel hands the rotated query between wavefronts through
 * LDS with bounded waits.  A wait that runs into its bound makes the workgroup publish NaN
 * partials (the output rows of that sequence come out NaN, not silently wrong) and raises a
 * device-side counter.  This call reads the counter of the current device since the library was
 * loaded; it synchronises with the device (it is a diagnostic, not part of a launch path).
 * Returns FQ_OK, or FQ_ERR_LAUNCH if the runtime refuses the copy.
 */
int fq_paged_decode_fault_count(unsigned int* count);

/* Number of splits fq_split_k_paged_decode uses when num_splits == 0, at
 * head_dim 128 (with 1 or 2 KV heads the other head dimensions run another
 * kernel and take another count)
 * (counterpart of paged_tq4_decode_num_splits, csrc/cuda/paged_decode.cu:424-426,
 * which is a constant 4 there). */
int fq_paged_decode_auto_splits(int num_seqs, int H_KV, int block_size,
                                int max_blocks_per_seq);

/* Smallest split count the decode kernel accepts for this context length: a
 * split may span at most 256 pages.  fq_split_k_paged_decode raises a smaller
 * request to this value; fq_paged_tq4_decode rejects it (FQ_ERR_BAD_SHAPE). */
int fq_paged_decode_min_splits(int block_size, int max_blocks_per_seq);

/* Bytes of workspace for the given launch; num_splits == 0 means "auto". */
size_t fq_paged_decode_workspace_bytes(int num_seqs, int H_Q, int H_KV, int D,
                                       int block_size, int max_blocks_per_seq,
                                       int num_splits);

/*
 * fq_split_k_paged_decode without a workspace argument and without any allocation.  It has no
 * counterpart in the reference; it is for callers that cannot call hipMalloc: code under HIP
 * graph capture, tight serving loops, harnesses that forbid allocation.  Arguments and results
 * are those of fq_split_k_paged_decode; the split partials and the rotated query live in an
 * array of FQ_STATIC_SCRATCH_BYTES bytes that the library keeps on every GPU it runs on until
 * the process ends.  A launch whose workspace (fq_paged_decode_workspace_bytes) exceeds that
 * size is refused with FQ_ERR_WORKSPACE.  All calls on one GPU share the array: calls that
 * overlap on one GPU (different streams, different threads) race; calls ordered on one stream
 * do not.  Calls no hipMalloc / hipFree; the first call on a device asks the runtime for the
 * array's address (hipGetSymbolAddress) and for the device's properties, and the first launch of
 * a kernel may make the runtime load its code: make one call on each device before a stream
 * capture begins (or in any other region where the runtime must not be asked for such things);
 * later calls on that device only launch kernels.
 */
#define FQ_STATIC_SCRATCH_BYTES (16u << 20)
size_t fq_static_scratch_bytes(void);
int fq_split_k_paged_decode_static(const void* q, const uint8_t* kv_cache,
                                   const int32_t* block_table, const int32_t* seq_lens,
                                   const float* centroids_k, const float* centroids_v,
                                   const float* rotation, int rotation_col_major, void* out,
                                   int num_seqs, int H_Q, int H_KV, int D,
                                   int block_size, int max_blocks_per_seq,
                                   int64_t num_blocks, float sm_scale, int dtype,
                                   int num_splits, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FQ_HIP_H */
