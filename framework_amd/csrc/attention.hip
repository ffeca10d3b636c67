// Softmax along one dim and the row kernels of attention built on the batched
// GEMM (scores = Q K^T, P = softmax(scale * scores [causal]), O = P V).
// Counterparts in the reference: ops/norm.rs:10-50, 96-123 (softmax and its
// backward) and ops/attention.rs:14-78, 143-202 (flash_attention and its
// backward), whose cuda arm (kernels/flash_attention.cu) walks the keys one by
// one per query row; here the two products run on the MFMA tile kernel and only
// the row-wise normalisation is left to these bandwidth kernels.
#include "common.h"

namespace mni {

static constexpr int ATT_TPB = 256;  // 4 wavefronts, one row each

static inline unsigned rows_grid(int64_t rows) { return (unsigned)((rows + 3) / 4); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// ---- softmax, contiguous lines (inner == 1): one wavefront per line -------------
__global__ void softmax_rows_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t rows, int64_t n) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *p = x + row * n;
    float *o = out + row * n;
    float mx = -INFINITY;
    for (int64_t j = lane; j < n; j += 64) mx = fmaxf(mx, p[j]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int64_t j = lane; j < n; j += 64) {
        const float e = expf(p[j] - mx);
        o[j] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    for (int64_t j = lane; j < n; j += 64) o[j] = o[j] / sum;
}
// lines with a stride (inner > 1): one thread per line, neighbours coalesce
__global__ void softmax_strided_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t outer, int64_t n,
                                       int64_t inner) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t base = (idx / inner) * n * inner + idx % inner;
    float mx = -INFINITY;
    for (int64_t t = 0; t < n; ++t) mx = fmaxf(mx, x[base + t * inner]);
    float sum = 0.f;
    for (int64_t t = 0; t < n; ++t) {
        const float e = expf(x[base + t * inner] - mx);
        out[base + t * inner] = e;
        sum += e;
    }
    for (int64_t t = 0; t < n; ++t) out[base + t * inner] /= sum;
}
int k_softmax(float *out, const float *x, int64_t outer, int64_t n, int64_t inner) {
    if (outer * n * inner <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (inner == 1)
        hipLaunchKernelGGL(softmax_rows_kernel, dim3(rows_grid(outer)), dim3(ATT_TPB), 0, ctx().stream, out, x, outer, n);
    else
        hipLaunchKernelGGL(softmax_strided_kernel, dim3((unsigned)((outer * inner + ATT_TPB - 1) / ATT_TPB)), dim3(ATT_TPB), 0,
                           ctx().stream, out, x, outer, n, inner);
    return check_launch("softmax");
}

// dx = sm * (g - sum(g * sm)) along the line
__global__ void softmax_bwd_rows_kernel(float *__restrict__ out, const float *__restrict__ sm, const float *__restrict__ g,
                                        int64_t rows, int64_t n) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *s = sm + row * n, *gr = g + row * n;
    float dot = 0.f;
    for (int64_t j = lane; j < n; j += 64) dot += gr[j] * s[j];
    dot = wave_sum(dot);
    for (int64_t j = lane; j < n; j += 64) out[row * n + j] = s[j] * (gr[j] - dot);
}
__global__ void softmax_bwd_strided_kernel(float *__restrict__ out, const float *__restrict__ sm,
                                           const float *__restrict__ g, int64_t outer, int64_t n, int64_t inner) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t base = (idx / inner) * n * inner + idx % inner;
    float dot = 0.f;
    for (int64_t t = 0; t < n; ++t) dot += g[base + t * inner] * sm[base + t * inner];
    for (int64_t t = 0; t < n; ++t) out[base + t * inner] = sm[base + t * inner] * (g[base + t * inner] - dot);
}
int k_softmax_backward(float *out, const float *sm, const float *g, int64_t outer, int64_t n, int64_t inner) {
    if (outer * n * inner <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (inner == 1)
        hipLaunchKernelGGL(softmax_bwd_rows_kernel, dim3(rows_grid(outer)), dim3(ATT_TPB), 0, ctx().stream, out, sm, g, outer, n);
    else
        hipLaunchKernelGGL(softmax_bwd_strided_kernel, dim3((unsigned)((outer * inner + ATT_TPB - 1) / ATT_TPB)), dim3(ATT_TPB),
                           0, ctx().stream, out, sm, g, outer, n, inner);
    return check_launch("softmax_backward");
}

// ---- attention rows -----------------------------------------------------------------
// scores[rows = bh * s][s] holds q.k; in place: P = softmax over the allowed
// columns of scale * scores (col <= row % s when causal), 0 elsewhere, and
// lse[row] = max + ln(sum) (ops/attention.rs:33-60).  One wavefront per row;
// rows of up to 1024 columns stay in registers between the passes.
__global__ void attn_softmax_kernel(float *__restrict__ scores, float *__restrict__ lse, int64_t rows, int s, float scale,
                                    int causal) {
    constexpr int R = 16;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    float *p = scores + row * (int64_t)s;
    const int col_end = causal ? (int)(row % s) + 1 : s;
    if (s <= 64 * R) {
        float v[R];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int j = lane + 64 * i;
            v[i] = j < col_end ? p[j] * scale : -INFINITY;
            mx = fmaxf(mx, v[i]);
        }
        mx = wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            v[i] = lane + 64 * i < col_end ? expf(v[i] - mx) : 0.f;
            sum += v[i];
        }
        sum = wave_sum(sum);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int j = lane + 64 * i;
            if (j < s) p[j] = v[i] * inv;
        }
        if (lane == 0) lse[row] = mx + logf(sum);
        return;
    }
    float mx = -INFINITY;
    for (int j = lane; j < col_end; j += 64) mx = fmaxf(mx, p[j] * scale);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int j = lane; j < col_end; j += 64) sum += expf(p[j] * scale - mx);
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    for (int j = lane; j < s; j += 64) p[j] = j < col_end ? expf(p[j] * scale - mx) * inv : 0.f;
    if (lane == 0) lse[row] = mx + logf(sum);
}
int k_attn_softmax(float *scores, float *lse, int64_t rows, int64_t s, float scale, int causal) {
    if (rows <= 0 || s <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    hipLaunchKernelGGL(attn_softmax_kernel, dim3(rows_grid(rows)), dim3(ATT_TPB), 0, ctx().stream, scores, lse, rows, (int)s,
                       scale, causal);
    return check_launch("attn_softmax");
}

// di[row] = sum_d a[row][d] * b[row][d] (ops/attention.rs:167-170)
__global__ void rowdot_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ b, int64_t rows,
                              int64_t d) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    float t = 0.f;
    for (int64_t j = lane; j < d; j += 64) t += a[row * d + j] * b[row * d + j];
    t = wave_sum(t);
    if (lane == 0) out[row] = t;
}
int k_rowdot(float *out, const float *a, const float *b, int64_t rows, int64_t d) {
    if (rows <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    hipLaunchKernelGGL(rowdot_kernel, dim3(rows_grid(rows)), dim3(ATT_TPB), 0, ctx().stream, out, a, b, rows, d);
    return check_launch("rowdot");
}

// In place over scores (q.k) and dp (dO.v), both [rows][s]:
//   P  = exp(scale * scores - lse[row]) on the allowed columns, 0 elsewhere
//   dS = P * (dp - di[row]) * scale                     (ops/attention.rs:172-187)
__global__ void attn_bwd_kernel(float *__restrict__ scores, float *__restrict__ dp, const float *__restrict__ lse,
                                const float *__restrict__ di, int64_t rows, int s, float scale, int causal) {
    const int64_t n = rows * (int64_t)s;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n; idx += step) {
        const int64_t row = idx / s;
        const int col = (int)(idx - row * s);
        const bool on = !causal || col <= (int)(row % s);
        const float p = on ? expf(scores[idx] * scale - lse[row]) : 0.f;
        scores[idx] = p;
        dp[idx] = p * (dp[idx] - di[row]) * scale;
    }
}
int k_attn_backward(float *scores, float *dp, const float *lse, const float *di, int64_t rows, int64_t s, float scale,
                    int causal) {
    const int64_t n = rows * s;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    int64_t blocks = (n + ATT_TPB * 4 - 1) / (ATT_TPB * 4);
    if (blocks > 65536) blocks = 65536;
    hipLaunchKernelGGL(attn_bwd_kernel, dim3((unsigned)blocks), dim3(ATT_TPB), 0, ctx().stream, scores, dp, lse, di, rows,
                       (int)s, scale, causal);
    return check_launch("attn_backward");
}

}  // namespace mni
