/*
 * mni_rocm.h -- C ABI of libmni_rocm.so, the MI355X (gfx950) backend for the
 * fp32 matrix-multiply path of mni-ml/framework.
 *
 * Two layers are exported:
 *
 *   1. Kernel level (mni_rocm_*): raw device pointers and sizes.  This is what
 *      a `rocm` cargo feature of the reference's Rust native layer binds with
 *      `extern "C"` from its own TensorStore/ops arms; each entry names the
 *      reference call site it replaces.
 *
 *   2. Engine level (mni_*): a self-contained counterpart of the reference's
 *      `Engine { store, tape }` behind its N-API bridge, one function per
 *      `#[napi]` export of src/native/src/lib.rs that the matmul path and its
 *      callers use.  Tensors are opaque u32 ids exactly as on the JS side.
 *
 * Conventions: no function throws or aborts.  Status-returning functions
 * return 0 on success and a non-zero MNI_ERR_* code on failure; id-returning
 * functions return MNI_BAD_ID on failure.  The message of the most recent
 * failure on the calling thread's library instance is available from
 * mni_rocm_last_error().  All work is issued on one library-owned HIP stream;
 * calls are stream-ordered, and only the documented functions synchronise.
 * The library is not re-entrant across threads (same contract as the
 * reference's single global mutex, src/native/src/lib.rs:27-39).
 */
#ifndef MNI_ROCM_H
#define MNI_ROCM_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MNI_OK 0
#define MNI_ERR_INVALID 1   /* bad argument / shape mismatch (reference: panic)   */
#define MNI_ERR_FREED 2     /* "tensor already freed" (src/native/src/tensor.rs:116) */
#define MNI_ERR_HIP 3       /* a HIP runtime call failed                           */
#define MNI_ERR_NOMEM 4     /* device allocation failed                            */
#define MNI_BAD_ID UINT32_MAX

/* ------------------------------------------------------------------------- *
 * 1. Kernel level
 * ------------------------------------------------------------------------- */

/* Device singleton: replaces GpuDevice::instance() of the cuda arm
 * (src/native/src/device.rs:29-48): one device, one stream, code objects
 * prebuilt into the library (no runtime compilation). Idempotent. */
int mni_rocm_init(int device);
/* Name reported by the HIP runtime and its compute-unit count / clock (kHz),
 * for roofline bookkeeping.  Any out pointer may be NULL. */
int mni_rocm_device_info(char *name, size_t name_cap, int *compute_units, int *clock_khz);
/* Number of XCDs (dies with an L2 of their own) that workgroups were seen to be
 * dealt over round-robin when the library started; 0 if that could not be
 * confirmed, in which case kernels that keep partial sums inside one XCD's L2
 * are not used.  < 0 on error.  No counterpart in the reference. */
int mni_rocm_device_xcds(void);
const char *mni_rocm_last_error(void);

/* Caching device allocator: replaces CachingAllocator of the cuda arm
 * (src/native/src/allocator.rs:46-84).  Exact-size free lists; unlike the
 * reference's cuda arm, memory handed to zero-initialised tensors is cleared
 * on reuse. */
int mni_rocm_malloc(void **ptr, size_t bytes);
int mni_rocm_free(void *ptr);
int mni_rocm_clear_cache(void);
/* Copies.  h2d/d2h synchronise the stream before returning (the reference's
 * memcpy_stod / memcpy_dtov, src/native/src/tensor.rs:364-387,460-469).
 * mni_rocm_sync, and mni_rocm_d2h of up to 16 KB, wait by queueing a small
 * kernel that writes a tag (and the data) to pinned host memory and watching
 * for it for up to 150 us, then fall back on hipStreamSynchronize: a wait
 * ends a few microseconds after the last kernel, and spins for that long at
 * most. */
int mni_rocm_h2d(void *dst, const void *src, size_t bytes);
int mni_rocm_d2h(void *dst, const void *src, size_t bytes);
int mni_rocm_d2d(void *dst, const void *src, size_t bytes);
int mni_rocm_sync(void);
/* Device status.  A kernel that has to wait for other workgroups of its own
 * launch (the single-launch K-slice reduction of the skinny kernel, the
 * stream-K tile fix-up, the decode product's partial sums) waits a bounded
 * number of polls; if the wait expires it writes NaN into the outputs
 * concerned and a code into a status word, and the next call that waits for
 * the stream (mni_rocm_sync, h2d, d2h, event_elapsed_ms and every engine call
 * built on them, such as mni_to_float32 / mni_get_scalar) returns MNI_ERR_HIP
 * with a message naming the kernel, and clears the word.  No counterpart in
 * the reference. */

/* Stream-ordered timing marks on the library's stream (HIP events). */
int mni_rocm_event_create(void **event);
int mni_rocm_event_record(void *event);
int mni_rocm_event_elapsed_ms(void *start, void *stop, float *ms); /* waits for stop */
int mni_rocm_event_destroy(void *event);

/* One operand of a product.  op(X) is addressed as
 *   X[batch b, row r, col c] = ptr[(b % batch_count) * batch_stride + r * row_stride + c * col_stride]
 * with strides in elements, so a transposed or permuted view is just a
 * different pair of strides: nothing is materialised.  `b % batch_count` is
 * the reference's batch rule (src/native/src/ops/matmul.rs:55-56). */
typedef struct {
    const float *ptr;
    int64_t row_stride;
    int64_t col_stride;
    int64_t batch_stride;
    int64_t batch_count; /* >= 1 */
} mni_operand;

/* NONE .. BIAS_GELU: C = f(product + bias).  The last two carry the fused Linear of a GELU layer through its
 * backward (the reference fuses bias + GELU and their backward outside the product, src/native/src/ops/fused.rs:247-351):
 *   BIAS_GELU_DUAL  C = product (the pre-activation without its bias, which the backward needs) and
 *                   aux = gelu(product + bias), written by the same epilogue;
 *   DGELU           C = product * gelu'(aux + bias) with aux the saved pre-activation, and, when colsum_part is
 *                   given, the column sums of C per strip of rows (summed afterwards: the bias gradient).
 * Both need `aux` laid out like C (same ldc and batch stride) and take no accumulate and no split_k. */
enum { MNI_EPI_NONE = 0, MNI_EPI_BIAS = 1, MNI_EPI_BIAS_RELU = 2, MNI_EPI_BIAS_GELU = 3, MNI_EPI_BIAS_GELU_DUAL = 4, MNI_EPI_DGELU = 5 };
/* MFMA = the MFMA tile kernel, one workgroup per tile and K slice, 128-wide tiles;
 * MFMA_SMALL = the same forced to 64 x 64 tiles; MFMA_STREAMK = the tile kernel
 * with the K steps of all tiles dealt evenly over a resident grid (error if the
 * device's workgroup-to-XCD mapping was not confirmed); SKINNY = the bandwidth
 * kernels (error if the shape or layout is not eligible); SKINNY_TWO_PASS = the
 * same with the K-slice partials summed by a second launch instead of inside
 * the first (SKINNY itself takes the second launch when the reducing
 * workgroups of the single launch would not all fit the device at once);
 * DIRECT = the register-direct MFMA kernel for batched products of
 * many small tiles (64 x 64 tiles, operands read from memory straight into the
 * matrix instruction's registers; split_k 0 or 1 = one wavefront per tile,
 * split_k 4 = four wavefronts sharing K; error if the operand layouts are not
 * eligible: each operand contiguous along K with K % 4 == 0, or along M / N
 * with that extent even); PANEL = the short-K kernel for two K-contiguous
 * operands (A row-major, B given as its transpose; K <= 64, K % 4 == 0; error
 * otherwise): 128 x 128 tiles, all of K at once, stores of one part of a tile
 * under the MFMAs of the next; TINY = one thread per output element and a
 * sequential sum over K, products rounded and added one by one as the
 * reference's CPU arm does (bit-identical to it), for products of a few
 * thousand outputs; FEWROWS = 9 to 32 rows of a K-contiguous A against a
 * wide N-contiguous B (a batch of token rows against a [in, out] weight): B
 * read once, straight into the matrix instruction's registers, K slices
 * (split_k, 0 = chosen) summed inside the launch (error unless K % 8 == 0,
 * N % 4 == 0, N >= 128, K >= 64, operands and C 16-byte aligned with row
 * strides in whole 16 bytes); OUTER = a short K (<= 512) under a large
 * output with A contiguous along M and B along N -- the weight gradient
 * X^T dY of a small batch: both operands straight into the matrix
 * instruction's registers, the cost of writing C (error unless N % 4 == 0,
 * B and C 16-byte aligned with row strides in whole 16 bytes, no epilogue;
 * accumulate is honoured); GEMV = the decode product, 1 to 32 rows of a
 * K-contiguous A against a row-major B that is as large as the product is
 * expensive: one workgroup per compute unit, a unit of columns and a K slice
 * each, the K slices summed inside the launch by whichever wavefront arrives
 * last.  Two forms: units of 128 columns for 1 to 8 rows, units of 64 for
 * up to 32 rows (A 16-byte aligned with a row stride in whole 16 bytes);
 * where both fit, the faster one is taken.  (Error unless one batch, N a
 * multiple of the unit with N / unit a divisor of the 256 compute units and
 * a multiple of 8, K a multiple of 512 (units of 128) or 1024 (units of 64)
 * times 256 / (N / unit), B, C and the bias 16-byte aligned with row strides
 * in whole 16 bytes, and no activation together with accumulate);
 * FEWROWS_NT = up to 32 rows of a
 * K-contiguous A against a wide B that is K-contiguous too (a weight stored
 * [out, in], given as its transposed view): a wavefront per 4 columns on
 * the 4 x 4 x 1 MFMA, A resident in LDS; with K up to 8192 / 4096 / 2048 /
 * 960 for up to 4 / 8 / 16 / 32 rows all of K per wavefront and no sums
 * across wavefronts, with a larger
 * K, or with a split_k of 2 to 16, K in that many slices of at most 1024
 * values (768 beyond 16 rows) that the last workgroup of a column block to
 * arrive adds up (error unless one batch, K % 64 == 0 and within those
 * limits, both operands 16-byte aligned with pitches in whole 16 bytes).
 * AUTO picks among them. */
enum { MNI_ALGO_AUTO = 0, MNI_ALGO_MFMA = 1, MNI_ALGO_SKINNY = 2, MNI_ALGO_MFMA_SMALL = 3, MNI_ALGO_SKINNY_TWO_PASS = 4,
       MNI_ALGO_MFMA_STREAMK = 5, MNI_ALGO_DIRECT = 6, MNI_ALGO_PANEL = 7, MNI_ALGO_TINY = 8, MNI_ALGO_FEWROWS = 9,
       MNI_ALGO_OUTER = 10, MNI_ALGO_GEMV = 11, MNI_ALGO_FEWROWS_NT = 12 };

/* C[b] (M x N, row stride ldc, unit column stride) = epilogue(op(A)[b] (M x K) * op(B)[b] (K x N)).
 * Replaces dev.blas.gemm / gemm_strided_batched (src/native/src/ops/matmul.rs:150-189),
 * the permute_f32 transposes feeding them (:287-326), the host gather of
 * non-contiguous operands (src/native/src/tensor.rs:510-517) and, with a bias
 * epilogue, add_bias_f32 (src/native/src/ops/elementwise.rs:105-130). */
typedef struct {
    int64_t M, N, K, batch;
    mni_operand A; /* op(A): rows = M, cols = K */
    mni_operand B; /* op(B): rows = K, cols = N */
    float *C;
    int64_t ldc;
    int64_t c_batch_stride;
    const float *bias;   /* N floats, or NULL when epilogue == MNI_EPI_NONE */
    int32_t epilogue;    /* MNI_EPI_*                                       */
    int32_t accumulate;  /* non-zero: C += result                            */
    int32_t split_k;     /* 0 = choose, 1 = never, n > 1 = exactly n slices */
    int32_t algo;        /* MNI_ALGO_*                                      */
    float *aux;          /* BIAS_GELU_DUAL: second output; DGELU: saved pre-activation (read); else NULL */
    float *colsum_part;  /* DGELU: mni_rocm_sgemm_colsum_rows(M, batch) x N floats of strip sums, or NULL */
} mni_gemm_desc;
int mni_rocm_sgemm(const mni_gemm_desc *desc);
/* Rows of the colsum_part matrix a DGELU product of this height and batch count writes. */
int64_t mni_rocm_sgemm_colsum_rows(int64_t M, int64_t batch);
/* The same product for callers that cannot allocate device memory (tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  The same kernels and the same sums as mni_rocm_sgemm, but the
 * partial sums of a split-K, stream-K or skinny plan go to a fixed 32 MiB
 * workspace that is part of the library's code object instead of a block
 * from the caching allocator, and nothing is allocated or freed during the
 * call.  Two differences in plan follow from that: a product whose B (or
 * ragged A) mni_rocm_sgemm would first repack into a scratch copy runs on
 * the operands as they are (same values, slower), and a product the decode
 * kernel would take keeps that kernel (its partial-sum slots are allocated at
 * mni_rocm_init).  The launches go to the library's own stream, as those of
 * every other entry point do: a caller cannot record them into a HIP graph
 * of its own.  Requires a prior mni_rocm_init (initialisation allocates;
 * this call refuses to initialise).  A product whose plan needs more than
 * mni_rocm_sgemm_noalloc_workspace_bytes() fails with MNI_ERR_INVALID and a
 * message giving both sizes (every plan the library chooses by itself fits;
 * an explicit split_k over a large C may not).  All calls share the one
 * workspace: they are ordered on the library's stream, so they do not race
 * with each other, but the workspace keeps the last call's partials and two
 * processes' or two libraries' calls on the same device memory would.
 * Nothing in it needs to start at zero. */
int mni_rocm_sgemm_noalloc(const mni_gemm_desc *desc);
size_t mni_rocm_sgemm_noalloc_workspace_bytes(void);
/* Two products that do not depend on each other: neither reads what the other
 * writes and their outputs do not overlap.  Replaces the two gemm calls of
 * matmul_backward (src/native/src/ops/matmul.rs:199-222: dA = dC * B^T and
 * dB = A^T * dC), which the reference issues one after the other.  When each
 * product alone is a batch of about one 64 x 64 tile per compute unit, both
 * run in one launch (every SIMD gets a second wavefront; one ramp-up, one
 * tail); so do two products of a few thousand outputs each (what
 * MNI_ALGO_AUTO gives to the tiny-product kernel: the gradients of a small
 * Linear); otherwise this is mni_rocm_sgemm(first) followed by
 * mni_rocm_sgemm(second).  The values are those of the separate calls within
 * the product's tolerance, and bit for bit wherever the separate call would
 * run the same kernel (the joint launches use the tile kernel's 64 x 64 tiles
 * in one K slice and the tiny-product kernel's sequential sum; a batch of
 * products against one shared B that mni_rocm_sgemm alone would fold into a
 * single tall product is summed in the unfolded order here). */
int mni_rocm_sgemm_pair(const mni_gemm_desc *first, const mni_gemm_desc *second);

/* dst (contiguous, `shape`) = gather of src by `src_strides` (elements).
 * Replaces permute_f32 (src/native/kernels/elementwise.cu:67-81) and the host
 * gather in ensure_contiguous (src/native/src/tensor.rs:510-517); up to 8 dims. */
int mni_rocm_strided_copy(float *dst, const float *src, const int64_t *shape,
                          const int64_t *src_strides, int ndim);
/* out[r, c] = a[r, c] + bias[c]   (add_bias_f32, src/native/kernels/elementwise.cu:43-47) */
int mni_rocm_add_bias(float *out, const float *a, const float *bias, int64_t rows, int64_t cols);
/* out[c] = sum_r a[r, c]          (bias gradient; replaces the host unbroadcast of
 * add_backward, src/native/src/ops/elementwise.rs:213-231) */
int mni_rocm_colsum(float *out, const float *a, int64_t rows, int64_t cols);
/* out (contiguous, `to_shape`) = g (contiguous, `g_shape`) summed over every dim that broadcasting `to_shape` up to
 * `g_shape` had stretched: the missing leading dims and every dim where to_shape is 1 and g_shape is not, interior
 * ones included ([2,3,M,K] -> [2,1,M,K]).  Each output is an f32 sum in the gradient's flat order.  Replaces
 * utils::unbroadcast (src/native/src/utils.rs:39-66) as matmul_backward (src/native/src/ops/matmul.rs:206-218) and
 * add_backward (src/native/src/ops/elementwise.rs:199-231) call it, which the reference's cuda arm runs on the host.
 * Equal shapes copy; up to 8 dims; error if the shapes do not broadcast. */
int mni_rocm_unbroadcast(float *out, const float *g, const int64_t *g_shape, int g_ndim, const int64_t *to_shape, int to_ndim);
/* dst[i] += alpha * src[i]        (add_f32 in accumulate_grad / add_inplace,
 * src/native/src/tensor.rs:475-508) */
int mni_rocm_axpy(float *dst, const float *src, float alpha, int64_t n);
/* dst[i] = value                  (fill_f32, src/native/src/tensor.rs:395-442) */
int mni_rocm_fill(float *dst, float value, int64_t n);

/* ------------------------------------------------------------------------- *
 * 2. Engine level: mirrors src/native/src/lib.rs export by export.
 * ------------------------------------------------------------------------- */

#define MNI_MAX_DIMS 8

uint32_t mni_zeros(const int64_t *shape, int ndim);                       /* lib.rs:45-50   */
uint32_t mni_ones(const int64_t *shape, int ndim);                        /* lib.rs:52-57   */
uint32_t mni_from_float32(const float *data, size_t len,
                          const int64_t *shape, int ndim);                /* lib.rs:73-78   */
int mni_tensor_shape(uint32_t id, int64_t *out, int cap);                 /* lib.rs:80-84; returns ndim or -1 */
int64_t mni_tensor_size(uint32_t id);                                     /* lib.rs:86-90   */
int mni_to_float32(uint32_t id, float *out, size_t cap);                  /* lib.rs:92-97   */
int mni_get_scalar(uint32_t id, double *out);                             /* lib.rs:99-103  */
void mni_free_tensor(uint32_t id);                                        /* lib.rs:105-109 */
int mni_set_requires_grad(uint32_t id, int requires);                     /* lib.rs:115-119 */
int mni_get_grad(uint32_t id, uint32_t *out);                             /* lib.rs:121-125; 1 = has grad, 0 = none, -1 = error */
int mni_backward(uint32_t loss);                                          /* lib.rs:131-137 */
int mni_zero_grad(const uint32_t *ids, size_t n);                         /* lib.rs:139-146 */
void mni_no_grad_start(void);                                             /* lib.rs:148-152 */
void mni_no_grad_end(void);                                               /* lib.rs:154-158 */
uint32_t mni_add(uint32_t a, uint32_t b);                                 /* lib.rs:164-169 */
uint32_t mni_mul(uint32_t a, uint32_t b);                                 /* lib.rs:171-176 */
uint32_t mni_sub(uint32_t a, uint32_t b);                                 /* lib.rs:178-183 */
uint32_t mni_neg(uint32_t a);                                             /* lib.rs:185-190 */
uint32_t mni_mul_scalar(uint32_t a, double s);                            /* lib.rs:192-197 */
uint32_t mni_matmul(uint32_t a, uint32_t b);                              /* lib.rs:199-204 */
uint32_t mni_gelu(uint32_t a);                                            /* lib.rs:206-211 */
uint32_t mni_relu(uint32_t a);                                            /* lib.rs:213-218 */
uint32_t mni_sum_op(uint32_t a, int64_t dim);                             /* lib.rs:234-239 */
uint32_t mni_mean_op(uint32_t a, int64_t dim);                            /* lib.rs:241-246 */
uint32_t mni_sum_all(uint32_t a);                                         /* lib.rs:255-265 */
uint32_t mni_mean_all(uint32_t a);                                        /* lib.rs:267-277 */
uint32_t mni_view(uint32_t a, const int64_t *shape, int ndim);            /* lib.rs:279-285 */
uint32_t mni_permute(uint32_t a, const int64_t *dims, int ndim);          /* lib.rs:287-293 */
uint32_t mni_contiguous(uint32_t a);                                      /* lib.rs:295-300 */
/* KV cache for incremental decoding (src/native/src/lib.rs:586-676 -> ops/kv_cache.rs): per cache
 * [batch * heads, max_seq_len, head_dim] keys and values in device memory, fp32 or int8 with one f32 scale per
 * row (quantize_row_i8, kv_cache.rs:357-370).  The reference keeps the cache in host memory and decodes on the
 * CPU; here append and decode are kernels.  Ids start at 1 and restart after mni_reset_engine.
 * create: new cache id, MNI_BAD_ID on error.  len / quantized: 0 for an unknown id.  reset / free: no-ops for
 * an unknown id.  append(k, v): k, v of shape [B,H,1,D] or [BH,1,D].  decode_step(q, k, v, scale): appends
 * k, v, then attends q over every cached position; returns the output tensor ([B,H,1,D] or [BH,1,D]).
 * Errors carry the reference's texts ("kv cache decode failed: kv cache decode expects seq_len=1, got 2", ...). */
uint32_t mni_kv_cache_create(int64_t batch_size, int64_t num_heads, int64_t head_dim, int64_t max_seq_len, int quantized);
int64_t mni_kv_cache_len(uint32_t cache_id);
int mni_kv_cache_quantized(uint32_t cache_id);
void mni_kv_cache_reset(uint32_t cache_id);
void mni_kv_cache_free(uint32_t cache_id);
int mni_kv_cache_append(uint32_t cache_id, uint32_t k, uint32_t v);
uint32_t mni_kv_cache_decode_step(uint32_t cache_id, uint32_t q, uint32_t k, uint32_t v, double scale);
/* Remaining elementwise / reduction exports of src/native/src/lib.rs, all on the device:
 * exp_op (:220-225), log_op (:227-232), sigmoid (:374-379), pow_op (:381-386; powf),
 * div (:339-344; broadcasting, backward da = g / b, db = -g a / b^2),
 * lt / eq_op / gt / is_close (:346-372; 1.0 or 0.0, nothing recorded),
 * max_op (:248-253; dim kept as size 1, the gradient goes to every element within 1e-6 of the maximum),
 * layernorm_op (:309-315; over the last extent, backward yields dx, dgamma, dbeta). */
uint32_t mni_exp_op(uint32_t a);
uint32_t mni_log_op(uint32_t a);
uint32_t mni_sigmoid(uint32_t a);
uint32_t mni_pow_op(uint32_t a, double exponent);
uint32_t mni_div(uint32_t a, uint32_t b);
uint32_t mni_lt(uint32_t a, uint32_t b);
uint32_t mni_eq_op(uint32_t a, uint32_t b);
uint32_t mni_gt(uint32_t a, uint32_t b);
uint32_t mni_is_close(uint32_t a, uint32_t b, double tol);
uint32_t mni_max_op(uint32_t a, int64_t dim);
uint32_t mni_layernorm_op(uint32_t x, uint32_t gamma, uint32_t beta, double eps);
/* Token side of a language-model step, device-resident.
 * rand_tensor / randn_tensor (src/native/src/lib.rs:60-71 -> tensor.rs:228-250): uniform [0, 1) in steps
 *   of 2^-24 and standard normal, drawn from a Philox4x32-10 stream on the device.  Like the reference's
 *   thread RNG the stream is seeded from system entropy; mni_seed (no counterpart in the reference) fixes
 *   it, and mni_philox_words exposes the raw generator (word i of the result is word i % 4 of block
 *   offset + i / 4 under key `seed`) so that it can be checked against the published test vectors.
 * dropout_op (lib.rs:388-394 -> ops/dropout.rs:25-58, backward :114-126): returns x itself when not
 *   training or rate == 0; else x * mask * 1/(1-rate) with mask = (u >= rate).  The mask is regenerated
 *   from the stream position in the backward instead of being stored.
 * create_dataset / sample_batch / free_int_buffer (lib.rs:476-497 -> ops/data.rs): int32 buffers in their
 *   own id space (LIFO recycling); sample_batch writes the ids of the inputs and targets buffers
 *   ([batch_size, block_size] windows at uniform starts in [0, len - block_size - 1), targets shifted by
 *   one) to out_ids[0..1].  mni_int_buffer_len / _to_host have no counterpart (the reference never reads
 *   these buffers back); they exist for tests and debugging.
 * embedding_forward (lib.rs:319-326 -> ops/embedding.rs:25-53) and embedding_forward_gpu (:501-511):
 *   out[b, t, :] = weight[index[b, t], :]; backward (:104-128) adds the gradient rows of equal indices
 *   in token order, on the device, deterministically.  Indices outside the table are an error.
 * cross_entropy_loss_gpu (lib.rs:679-691 -> ops/loss.rs:190-229): logits viewed as [rows, classes],
 *   targets taken from an int buffer.
 * residual_layernorm (lib.rs:515-523 -> ops/fused.rs:23-78, backward :134-186): layernorm(x + residual)
 *   in one pass; x and residual receive the same gradient tensor.
 * scale_grads (lib.rs:450-454 -> ops/mixed_precision.rs:17-32): grads *= inv_scale; *found_inf = 1 when
 *   any scaled value is infinite or NaN.
 * tile (lib.rs:568-573 -> ops/pooling.rs:276-309): repeat along every dim; not differentiable. */
uint32_t mni_rand_tensor(const int64_t *shape, int ndim);
uint32_t mni_randn_tensor(const int64_t *shape, int ndim);
int mni_seed(uint64_t seed);
int mni_philox_words(uint64_t seed, uint64_t offset, uint32_t *out, size_t n);
uint32_t mni_dropout_op(uint32_t x, double rate, int training);
uint32_t mni_create_dataset(const int32_t *data, size_t len);
int mni_sample_batch(uint32_t dataset, int64_t block_size, int64_t batch_size, uint32_t *out_ids);
int mni_free_int_buffer(uint32_t id);
int64_t mni_int_buffer_len(uint32_t id); /* < 0 on error */
int mni_int_buffer_to_host(uint32_t id, int32_t *out, size_t cap);
uint32_t mni_embedding_forward(uint32_t weight, const int64_t *indices, size_t n, int64_t batch, int64_t seq_len);
uint32_t mni_embedding_forward_gpu(uint32_t weight, uint32_t int_buf, int64_t batch, int64_t seq_len);
uint32_t mni_cross_entropy_loss_gpu(uint32_t logits, uint32_t int_buf);
uint32_t mni_residual_layernorm(uint32_t x, uint32_t residual, uint32_t gamma, uint32_t beta, double eps);
int mni_scale_grads(const uint32_t *ids, size_t n, double inv_scale, int *found_inf);
uint32_t mni_tile(uint32_t input, const int64_t *reps, int n);
/* bias_gelu (src/native/src/lib.rs:526-531 -> ops/fused.rs:247-273, backward :316-351):
 * out = gelu(x + bias) along the last extent; backward yields dx and the column sums dbias in one pass. */
uint32_t mni_bias_gelu(uint32_t x, uint32_t bias);
/* softmax_op (src/native/src/lib.rs:302-307 -> ops/norm.rs:10-50); backward as
 * ops/norm.rs:96-123, including its reading of a negative saved dim as dim 0. */
uint32_t mni_softmax_op(uint32_t a, int64_t dim);
/* flash_attention (src/native/src/lib.rs:575-584 -> ops/attention.rs:14-78,
 * backward :143-202): q, k, v taken as [bh, s, d] from their first three dims;
 * returns out [bh, s, d].  Head dims 32, 64, 96 and 128 run the forward in one
 * MFMA kernel and the backward in two (scores and probabilities never reach
 * memory); other head dims are built on the batched GEMM (q k^T, P v and the
 * five backward products) with row kernels for scale / causal mask /
 * normalisation.  Either replaces the per-key loop of kernels/flash_attention.cu. */
uint32_t mni_flash_attention(uint32_t q, uint32_t k, uint32_t v, double scale, int causal);
uint32_t mni_cross_entropy_loss(uint32_t logits, const int64_t *targets, size_t n); /* lib.rs:328-336 */
int mni_adamw_step(const uint32_t *ids, size_t n, double lr, double beta1, double beta2,
                   double eps, double weight_decay, int64_t step);        /* lib.rs:400-412 */
double mni_grad_norm(const uint32_t *ids, size_t n);                      /* lib.rs:414-419; < 0 on error */
int mni_clip_grad_norm(const uint32_t *ids, size_t n, double max_norm);   /* lib.rs:421-426 */
double mni_clip_and_step(const uint32_t *ids, size_t n, double lr, double beta1, double beta2,
                         double eps, double weight_decay, int64_t step,
                         double max_grad_norm);                           /* lib.rs:428-442; < 0 on error */
void mni_reset_engine(void);                                              /* lib.rs:460-468 */
int mni_gc_tensors(const uint32_t *keep, size_t n);                       /* lib.rs:693-706 */

/* Opt-in fused Linear: out = x * w + bias in one product with a bias
 * epilogue, recorded as one tape entry whose backward yields dX, dW and db.
 * The reference composes this from `matmul` then `add` (src/nn.ts:23-25); a
 * caller feature-detects this export the way the reference detects its
 * cuda-only fused ops (src/nn.ts:116, test/native.test.ts:13).
 * act: MNI_EPI_BIAS (none), MNI_EPI_BIAS_RELU or MNI_EPI_BIAS_GELU. */
uint32_t mni_linear(uint32_t x, uint32_t w, uint32_t bias, int act);

/* Opt-in fused mseLoss: what src/nn.ts:161-165 composes from sub, mul and two
 * mean(-1) calls, in one pass and one tape entry whose backward is one pass
 * too.  Same result as the composition: one mean of squared differences per
 * row of the last dim, shape [..., 1] (the composition's second mean runs
 * over the size-1 dim the first one leaves).  Shapes must be equal; a caller
 * that needs broadcasting keeps the composition.  Feature-detected like
 * mni_linear. */
uint32_t mni_mse_loss(uint32_t pred, uint32_t target);

/* Device address of a tensor's buffer (cuda arm: TensorStore::dev_ptr,
 * src/native/src/tensor.rs:358-361). NULL on error. */
void *mni_dev_ptr(uint32_t id);

/* ------------------------------------------------------------------------- *
 * Measurement and test hooks.  NOT part of the drop-in boundary: nothing the
 * reference binds has a counterpart here and an integration needs none of
 * them.  They exist so that benchmarks can issue launches from C (the host
 * stays ahead of kernels of a few microseconds), so that a kernel can be held
 * against what the device gives a loop that only streams or only issues
 * MFMAs, and so that tests can reach an error path without hanging a kernel.
 * ------------------------------------------------------------------------- */
/* Sets the device status word from the host, as a kernel whose bounded wait
 * expired would: the next call that waits for the stream reports it. */
int mni_rocm_test_raise_device_status(unsigned code);

/* Kernels launched by the library since it was loaded (copies not counted):
 * what a latency-bound training step is made of. */
uint64_t mni_rocm_launch_count(void);

/* The library's device allocator since it was loaded: requests made of it
 * (mni_rocm_malloc, tensors, workspaces), those that went on to hipMalloc
 * (the others were served from its free lists), blocks given back to it, and
 * the bytes its free lists hold now.  A test of mni_rocm_sgemm_noalloc reads
 * them before and after the call. */
int mni_rocm_alloc_stats(uint64_t *requests, uint64_t *driver_allocations, uint64_t *releases, uint64_t *cached_bytes);

/* Runs descs[0], descs[1],
 * ... descs[count-1], descs[0], ... back to back on the library's stream,
 * `warmup` untimed launches and then `iters` launches between two HIP events,
 * and returns the average milliseconds per launch.  Issuing from C keeps the
 * host ahead of kernels that take only a few microseconds. */
int mni_rocm_sgemm_timed(const mni_gemm_desc *descs, int count, int warmup, int iters, float *avg_ms);
/* The same for mni_rocm_sgemm_pair: descs holds count / 2 pairs (descs[0] with
 * descs[1], descs[2] with descs[3], ...); the average is per pair. */
int mni_rocm_sgemm_pair_timed(const mni_gemm_desc *descs, int count, int warmup, int iters, float *avg_ms);
/* What the device gives a
 * kernel that only streams.  `iters` launches between two HIP events on the
 * library's stream after `warmup` untimed ones; the average milliseconds per
 * launch is returned.  EMPTY: a one-wavefront kernel that does nothing (the
 * cost of a launch in a back-to-back sequence).  READ: `bytes` bytes of
 * srcs[launch % nsrc] are read with 16-byte loads, 8 in flight per lane, and
 * nothing is written (several sources in rotation make the pass cold in the
 * last-level cache).  WRITE: `bytes` bytes of dst are written.  COPY: both.
 * `nontemporal` selects streaming loads / stores; the grid is blocks_per_cu
 * workgroups of 256 threads per compute unit.  Sizes are multiples of 16. */
enum { MNI_YARDSTICK_EMPTY = 0, MNI_YARDSTICK_READ = 1, MNI_YARDSTICK_WRITE = 2, MNI_YARDSTICK_COPY = 3 };
int mni_rocm_yardstick_timed(int kind, int nontemporal, void *dst, const void *const *srcs, int nsrc, size_t bytes,
                             int blocks_per_cu, int warmup, int iters, float *avg_ms);
/* What the matrix pipe
 * gives a loop of nothing but fp32 MFMAs.  Every wavefront issues
 * `mfmas_per_wave` (a multiple of 16) v_mfma_f32_32x32x2_f32 on four
 * independent accumulators, each followed by `valu_per_mfma` (0..2) v_mov_b32
 * that depend on nothing; the grid is `waves_per_simd` (1 or 2) workgroups of
 * four wavefronts per compute unit.  Returns the average milliseconds per
 * launch; the rate is CUs * 4 * waves_per_simd * mfmas_per_wave * 4096 flop
 * over that.  The figure with valu_per_mfma = 0 is the ceiling an MFMA-bound
 * product is held against next to the datasheet's; the others show what every
 * vector-ALU instruction inside an MFMA loop costs on this device. */
int mni_rocm_mfma_yardstick_timed(int valu_per_mfma, int waves_per_simd, int mfmas_per_wave, int warmup, int iters, float *avg_ms);

#ifdef __cplusplus
}
#endif
#endif /* MNI_ROCM_H */
