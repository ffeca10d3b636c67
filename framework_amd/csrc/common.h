// Shared declarations of libmni_rocm.so: device context, allocator, error
// reporting and the internal launchers the C ABI and the engine are built on.
#pragma once
#include <mutex>

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/mni_rocm.h"

namespace mni {

// ---- error reporting -------------------------------------------------------
int set_error(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

#define MNI_HIP_CHECK(expr)                                                              \
    do {                                                                                 \
        hipError_t e_ = (expr);                                                          \
        if (e_ != hipSuccess)                                                            \
            return ::mni::set_error(MNI_ERR_HIP, "%s failed: %s (%s:%d)", #expr,         \
                                    hipGetErrorString(e_), __FILE__, __LINE__);          \
    } while (0)

#define MNI_TRY(expr)              \
    do {                           \
        int rc_ = (expr);          \
        if (rc_ != MNI_OK) return rc_; \
    } while (0)

// ---- device context --------------------------------------------------------
struct DeviceCtx {
    bool ready = false;
    int device = 0;
    int compute_units = 0;
    int clock_khz = 0;
    char name[256] = {0};
    hipStream_t stream = nullptr;
    // Workgroup b of a 1-D grid runs on XCD b % xcd_count when the start-up
    // probe confirmed it (0 = not confirmed; kernels that rely on sharing one
    // XCD's L2 are then not used).
    int xcd_count = 0;
    // Arrival flags of the single-launch skinny kernel: [unit][slice], each
    // launch marks them with a fresh epoch so they never need clearing.
    unsigned *skinny_flags = nullptr;
    size_t skinny_flag_cap = 0;  // entries
    // Arrival counters of the few-rows kernel's K slices, one per (batch, column group); zero between launches.
    unsigned *fewrows_counters = nullptr;
    size_t fewrows_counter_cap = 0;
    unsigned skinny_epoch = 0;
    // K-slice partials and arrival counters of the decode product (gemv_units_kernel): the partials carry the
    // launch's epoch as a tag, so the buffer is written by that kernel alone and by nothing else, ever.
    void *gemv_pa = nullptr;  // gemv_slot_cap pieces of 16 bytes
    void *gemv_pb = nullptr;  // gemv_slot_cap pieces of 8 bytes
    size_t gemv_slot_cap = 0;
    unsigned *gemv_counters = nullptr;
    size_t gemv_counter_cap = 0;
    // Device status word in pinned host memory that kernels can write: a kernel
    // whose bounded wait for another workgroup expires stores a DEVICE_STATUS_*
    // code there (and NaN into its outputs).  Every call that waits for the
    // stream reads the word afterwards and fails loudly when it is set.
    unsigned *status_host = nullptr;  // host address
    unsigned *status_dev = nullptr;   // the same word as kernels address it
    // A second word in the same pinned block: a kernel leaves a 32-bit result there, tagged with the number
    // the host gave it, and the host reads it without a copy or a wait for the stream (wait_result_word).
    unsigned long long *result_host = nullptr;
    unsigned long long *result_dev = nullptr;
    unsigned result_seq = 0;
    // Pinned, device-visible buffer that small device-to-host reads arrive in (mni_rocm_d2h).
    unsigned *fetch_host = nullptr;
    unsigned *fetch_dev = nullptr;
    // Workspace source of the current sgemm call: null = the caching allocator;
    // otherwise the product's partial sums are placed in this preallocated
    // block of `scratch_bytes` (the entry point that must not allocate).
    float *scratch = nullptr;
    size_t scratch_bytes = 0;
    // Kernels launched since the library was loaded (bookkeeping for latency-bound steps).
    uint64_t launches = 0;
    // Device address and size of the library's static workspace (see device.hip).
    float *noalloc_scratch = nullptr;
    size_t noalloc_scratch_bytes = 0;
    // Pinned staging slots for small host-to-device uploads that must not stall the host (upload_small).
    static constexpr int STAGE_SLOTS = 16;
    static constexpr size_t STAGE_BYTES = 16384;
    char *stage_host = nullptr;            // STAGE_SLOTS x STAGE_BYTES, pinned
    hipEvent_t stage_done[STAGE_SLOTS] = {};
    bool stage_used[STAGE_SLOTS] = {};
    unsigned stage_next = 0;
};
// Host-to-device upload of `bytes` bytes on the library's stream.  Up to STAGE_BYTES the data is copied into a
// pinned staging slot and the transfer is only enqueued: the host does not wait for the stream (an ordinary
// mni_rocm_h2d drains everything queued so far), and `src` may be reused at once.  Larger uploads wait.
int upload_small(void *dst, const void *src, size_t bytes);
// A kernel hands one 32-bit value to the host: next_result_tag() clears the result word and returns the tag for
// the launch; the kernel's last act is one 8-byte store of (tag << 32 | value) to ctx().result_dev;
// wait_result_word() returns the value once that store has arrived.  It watches the word for a short while
// (a kernel that is next in line delivers within microseconds), then waits for the stream; false in *delivered
// if even then the word has not come (the caller has another way to the value).
#ifdef __HIPCC__
// One 8-byte store to pinned host memory: the host sees the tag and the value together or not at all.  Relaxed: a
// release at system scope would write the whole L2 back first (microseconds, with the host waiting); a kernel that
// hands over more than the word fences what it wrote itself (fetch_small_kernel).
__device__ __forceinline__ void post_result_word(unsigned long long *word, unsigned tag, unsigned value) {
    __hip_atomic_store(word, ((unsigned long long)tag << 32) | (unsigned long long)value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}
// One workgroup (blockDim.x threads, whole wavefronts, at most 1024) turns one contiguous line of n values into its
// softmax, o[j] = exp(p[j] - max) / sum, in three passes over the line (the second and third re-read what the
// workgroup itself touched: L2), and hands max and sum to every thread.  `vec`: n % 4 == 0 and both lines 16-byte
// aligned.  `red`: 32 floats of LDS.  Sums are taken per thread, then per wavefront, then in wavefront order.
__device__ __forceinline__ void softmax_line_workgroup(float *__restrict__ o, const float *__restrict__ p, int64_t n, bool vec,
                                                       float *red, float &mx_out, float &sum_out) {
    const int tid = threadIdx.x, nt = blockDim.x, lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
    const int64_t n4 = n >> 2;
    const float4 *p4 = reinterpret_cast<const float4 *>(p);
    float4 *o4 = reinterpret_cast<float4 *>(o);
    float mx = -INFINITY;
    if (vec) {
        for (int64_t j = tid; j < n4; j += nt) {
            const float4 v = p4[j];
            mx = fmaxf(fmaxf(mx, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
        }
    } else {
        for (int64_t j = tid; j < n; j += nt) mx = fmaxf(mx, p[j]);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    mx = red[0];
    for (int w = 1; w < nw; ++w) mx = fmaxf(mx, red[w]);
    float sum = 0.f;
    if (vec) {
        for (int64_t j = tid; j < n4; j += nt) {
            float4 v = p4[j];
            v.x = expf(v.x - mx); v.y = expf(v.y - mx); v.z = expf(v.z - mx); v.w = expf(v.w - mx);
            o4[j] = v;
            sum += v.x; sum += v.y; sum += v.z; sum += v.w;
        }
    } else {
        for (int64_t j = tid; j < n; j += nt) {
            const float e = expf(p[j] - mx);
            o[j] = e;
            sum += e;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) red[16 + wave] = sum;
    __syncthreads();
    sum = red[16];
    for (int w = 1; w < nw; ++w) sum += red[16 + w];
    if (vec) {
        for (int64_t j = tid; j < n4; j += nt) {
            float4 v = o4[j];  // (written by this thread)
            o4[j] = make_float4(v.x / sum, v.y / sum, v.z / sum, v.w / sum);
        }
    } else {
        for (int64_t j = tid; j < n; j += nt) o[j] = o[j] / sum;
    }
    mx_out = mx;
    sum_out = sum;
}
#endif
unsigned next_result_tag();
int wait_result_word(unsigned tag, unsigned *value, bool *delivered);
enum { DEVICE_STATUS_OK = 0, DEVICE_STATUS_STREAMK_WAIT = 1, DEVICE_STATUS_SKINNY_WAIT = 2, DEVICE_STATUS_GEMV_WAIT = 3 };
// hipStreamSynchronize on the library's stream, then the device status word:
// MNI_ERR_HIP naming the kernel when a bounded wait expired since the last check.
int sync_stream_checked(const char *what);
// The status word alone, for callers that have already waited (on an event).
int check_device_status(const char *what);
// Workspace of one product: from ctx().scratch when set (error when `bytes`
// exceeds it), else from the caching allocator.  Release with gemm_ws_free.
int gemm_ws_alloc(void **p, size_t bytes);
void gemm_ws_free(void *p);
DeviceCtx &ctx();

// Every extern "C" entry point holds this for its whole duration: the engine
// and the allocator are single-threaded by design, as the reference's Engine
// behind its one mutex is (src/native/src/lib.rs:27-39).  Recursive because
// engine-level entry points call kernel-level ones.
std::recursive_mutex &api_mutex();
#define MNI_API_GUARD std::lock_guard<std::recursive_mutex> mni_api_guard_(mni::api_mutex())
int ensure_init();  // initialises device 0 on first use

// ---- caching allocator -----------------------------------------------------
int dev_alloc(void **p, size_t bytes);  // contents undefined
int dev_free(void *p);
int dev_clear_cache();
size_t dev_cached_bytes();  // bytes held in free lists
void dev_alloc_stats(uint64_t *requests, uint64_t *driver_allocations, uint64_t *releases, uint64_t *cached_bytes);

// ---- launch helpers --------------------------------------------------------
// Every kernel launch of the library goes through this, so that launches can be counted.
#define MNI_KERNEL_LAUNCH(...)          \
    do {                                \
        ++::mni::ctx().launches;        \
        hipLaunchKernelGGL(__VA_ARGS__); \
    } while (0)
int check_launch(const char *what);  // hipGetLastError after a kernel launch

// gemm.hip
int sgemm(const mni_gemm_desc &d);
// Two independent products, in one launch where the paired tile kernel takes them (gemm.hip).
// `colsum` (may be null): column sums the caller needs as well (a Linear's bias gradient); computed in the same launch
// when the pair goes out as one launch of the tiny-product kernel and the matrix is small, and colsum->done says so.
struct PairColsum;
int sgemm_pair(const mni_gemm_desc &d0, const mni_gemm_desc &d1, PairColsum *colsum = nullptr);

// elementwise.hip: internal launchers (device pointers, element strides)
struct StridedDesc {
    int ndim;
    int64_t shape[MNI_MAX_DIMS];
    int64_t a_strides[MNI_MAX_DIMS];
    int64_t b_strides[MNI_MAX_DIMS];
};
enum BinOp { BIN_ADD = 0, BIN_SUB = 1, BIN_MUL = 2, BIN_DIV = 3, BIN_LT = 4, BIN_EQ = 5, BIN_GT = 6, BIN_CLOSE = 7 };
enum UnOp { UN_RELU = 0, UN_GELU = 1, UN_NEG = 2, UN_SCALE = 3, UN_COPY = 4, UN_EXP = 5, UN_LOG = 6, UN_SIGMOID = 7, UN_POW = 8 };

int k_fill(float *dst, float v, int64_t n);
int k_axpy(float *dst, const float *src, float alpha, int64_t n);
int k_scale_inplace(float *dst, float s, int64_t n);
int k_strided_copy(float *dst, const float *src, const int64_t *shape, const int64_t *strides, int ndim);
// `p` is the tolerance of BIN_CLOSE (|a - b| < p)
int k_binary_broadcast(float *out, const float *a, const float *b, const StridedDesc &d, int op, float p = 0.f);
int k_binary_same(float *out, const float *a, const float *b, int64_t n, int op, float p = 0.f);
// ga = g / b, gb = -g * a / (b * b); g contiguous over d.shape, a / b addressed by d.a_strides / d.b_strides
int k_div_backward(float *ga, float *gb, const float *g, const float *a, const float *b, const StridedDesc &d);
int k_add_bias(float *out, const float *a, const float *bias, int64_t rows, int64_t cols);
int k_unary(float *out, const float *x, int64_t n, int op, float s);
// out = g * f'(x) for relu/gelu
int k_unary_backward(float *out, const float *g, const float *x, int64_t n, int op);
// exp: g * out, log: g / x, sigmoid: g * o * (1 - o), pow: g * s * x^(s - 1); `saved` is out or x accordingly
int k_unary2_backward(float *out, const float *g, const float *saved, int64_t n, int op, float s);
int k_mul_backward_same(float *ga, float *gb, const float *g, const float *a, const float *b, int64_t n);
int k_colsum(float *out, const float *a, int64_t rows, int64_t cols);
// out[o, i] = (sum_d a[o, d, i]) / div
int k_reduce_dim(float *out, const float *a, int64_t outer, int64_t dim, int64_t inner, float div);
// layernorm (residual == nullptr) or residual + layernorm of rows of 1024 to 16384 values, a workgroup per row;
// false (nothing launched) when the rows do not fit that form
bool launch_layernorm_workgroups(float *out, float *res, float *mean, float *rstd, const float *x, const float *residual,
                                 const float *gamma, const float *beta, int64_t rows, int64_t c, float eps);
// out[o, d, i] = g[o, i] / div
int k_expand_dim(float *out, const float *g, int64_t outer, int64_t dim, int64_t inner, float div);
// generic unbroadcast: out (orig shape, contiguous) = sum of g over broadcast dims
int k_unbroadcast(float *out, const float *g, const int64_t *gshape, int gnd, const int64_t *oshape, int ond);
// targets: device buffer of n values.  targets_host: null when `targets` already holds them; otherwise the values
// (each in [0, v)), which the call brings to `targets` itself.
// grad_for_one (may be null): n * v floats; a small batch's launch also leaves there the gradient of the logits for
// an upstream gradient of exactly one, and *wrote_grad says whether it did.
int k_cross_entropy(float *loss, float *softmax, const float *logits, int32_t *targets, const int32_t *targets_host,
                    int64_t n, int64_t v, float *grad_for_one = nullptr, bool *wrote_grad = nullptr);
// out[r] = mean_c (p - t)^2 and its backward (dt may be null)
int k_mse_rows(float *out, const float *p, const float *t, int64_t rows, int64_t dim, float *seeded = nullptr);  // seeded: also the gradient for an upstream gradient of ones
int k_mse_rows_backward(float *dp, float *dt, const float *p, const float *t, const float *g, int64_t rows, int64_t dim);
int k_cross_entropy_backward(float *dlogits, const float *softmax, const int32_t *targets,
                             const float *grad_scalar, int64_t n, int64_t v);
int k_bias_gelu(float *out, const float *x, const float *bias, int64_t rows, int64_t cols);
int k_bias_gelu_backward(float *dx, float *dbias, const float *g, const float *x, const float *bias, int64_t rows,
                         int64_t cols);
// out[o, i] = max_d a[o, d, i]; backward: g[o, i] where |x - max| < 1e-6, else 0
int k_max_dim(float *out, const float *a, int64_t outer, int64_t dim, int64_t inner);
int k_max_backward(float *out, const float *x, const float *mx, const float *g, int64_t outer, int64_t dim, int64_t inner);
int k_layernorm(float *out, float *mean, float *rstd, const float *x, const float *gamma, const float *beta, int64_t rows,
                int64_t c, float eps);
int k_layernorm_backward(float *dx, float *dgamma, float *dbeta, const float *g, const float *x, const float *gamma,
                         const float *mean, const float *rstd, int64_t rows, int64_t c);
// attention.hip
int k_softmax(float *out, const float *x, int64_t outer, int64_t n, int64_t inner);
int k_softmax_backward(float *out, const float *sm, const float *g, int64_t outer, int64_t n, int64_t inner);
int k_attn_softmax(float *scores, float *lse, int64_t rows, int64_t s, float scale, int causal);
int k_rowdot(float *out, const float *a, const float *b, int64_t rows, int64_t d);
// Attention forward in one kernel (out [bh,s,d], lse [bh,s]); head dims 32, 64, 96, 128 only.
bool attn_fused_supported(int64_t d);
int k_attn_fused_forward(float *out, float *lse, const float *q, const float *k, const float *v, int64_t bh, int64_t s, int64_t d,
                         float scale, int causal);
// dq of the attention backward in one kernel (same head dims); di[row] = sum_d dO * O.
int k_attn_fused_backward_dq(float *dq, const float *q, const float *k, const float *v, const float *dout, const float *lse,
                             const float *di, int64_t bh, int64_t s, int64_t d, float scale, int causal);
int k_attn_fused_backward_dkv(float *dk, float *dv, const float *q, const float *k, const float *v, const float *dout,
                              const float *lse, const float *di, int64_t bh, int64_t s, int64_t d, float scale, int causal);
int k_attn_backward(float *scores, float *dp, const float *lse, const float *di, int64_t rows, int64_t s, float scale,
                    int causal);
int k_kv_append(void *kc, void *vc, float *ks, float *vs, const float *k, const float *v, int64_t bh, int64_t d,
                int64_t max_seq, int64_t pos, int quantized);
int k_kv_decode(float *out, const void *kc, const void *vc, const float *ks, const float *vs, const float *q, int64_t bh,
                int64_t d, int64_t max_seq, int64_t len, float scale, int quantized);

// sequence.hip
// mode 0: uniform [0, 1), 1: standard normal, 2: the raw Philox words; element i is word i % 4 of block offset + i / 4
int k_random_fill(float *out, int64_t n, uint64_t seed, uint64_t offset, int mode);
// out = x * (u >= rate) * scale with the uniforms of (seed, offset); also the backward, with the gradient as x
int k_dropout(float *out, const float *x, int64_t n, float rate, float scale, uint64_t seed, uint64_t offset);
int k_sample_windows(int32_t *inputs, int32_t *targets, const int32_t *data, const int32_t *starts, int64_t block, int64_t batch);
int k_embedding_forward(float *out, const float *w, const int32_t *idx, int64_t tokens, int64_t dim);
// dw[v] = sum of g[t] over idx[t] == v in increasing t; `work` holds 3 * vocab + 2 + 2 * tokens int32 values
int k_embedding_backward(float *dw, const float *g, const int32_t *idx, int64_t tokens, int64_t vocab, int64_t dim,
                         int32_t *work);
int k_tile(float *out, const float *in, const int64_t *in_shape, const int64_t *reps, int ndim);
int k_residual_layernorm(float *out, float *res, float *mean, float *rstd, const float *x, const float *residual,
                         const float *gamma, const float *beta, int64_t rows, int64_t c, float eps);
// g *= s; *flag = 1 if any scaled value is infinite or NaN (flag is not cleared here)
int k_scale_check(float *g, float s, int64_t n, float *flag);

int k_sumsq_f64(double *out, const float *g, int64_t n);  // out += sum g^2 (device double)
// The same in two steps, so that many tensors share one final sum: partials of
// one tensor (sumsq_blocks(n) doubles), then out += sum of all partials.
int sumsq_blocks(int64_t n);
int k_sumsq_partials(double *part, const float *g, int64_t n);
// result_word / tag: when given, (float)out[0] also goes to that word (see wait_result_word).
int k_sumsq_finish(double *out, const double *part, int nparts, bool overwrite = false, unsigned long long *result_word = nullptr,
                   unsigned tag = 0);
int k_adamw(float *p, float *m, float *v, const float *g, int64_t n, float lr, float b1, float b2,
            float eps, float wd, float bc1, float bc2);
// Many tensors in one launch.  Tensor i owns workgroups [block_start[i], block_start[i + 1]), one per
// MULTI_CHUNK elements (multi_tensor_blocks(n[i]) of them).  k_sumsq_multi writes one partial per workgroup.
constexpr int MULTI_MAX = 48;
constexpr int MULTI_CHUNK = 4096;
struct MultiTensor {
    int count;
    int block_start[MULTI_MAX + 1];
    float *p[MULTI_MAX], *m[MULTI_MAX], *v[MULTI_MAX];
    const float *g[MULTI_MAX];
    int64_t n[MULTI_MAX];
};
int multi_tensor_blocks(int64_t n);
int k_adamw_multi(const MultiTensor &t, float lr, float b1, float b2, float eps, float wd, float bc1, float bc2);
int k_sumsq_multi(const MultiTensor &t, double *part);
// Up to SUMSQ_SOLO_BLOCKS workgroups' worth of gradients: one workgroup computes the partial sums one after the
// other and adds them up, in the order of k_sumsq_multi + k_sumsq_finish (same value); out[0] = the sum.
constexpr int SUMSQ_SOLO_BLOCKS = 16;
int k_sumsq_solo(const MultiTensor &t, double *out, unsigned long long *result_word, unsigned tag);
// The same launch then clips the gradients in place (norm > max_norm > 0) and applies AdamW to every tensor of the table.
int k_clip_and_step_solo(const MultiTensor &t, double *out, unsigned long long *result_word, unsigned tag, float max_norm, float lr, float b1,
                         float b2, float eps, float wd, float bc1, float bc2);

}  // namespace mni
