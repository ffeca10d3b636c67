// Token-side kernels of a language-model training step, so that no part of it
// goes through host memory: device-resident token datasets and batch windows
// (src/native/src/ops/data.rs), the embedding gather and its scatter-add in
// token order (ops/embedding.rs), counter-based random numbers for rand /
// randn / dropout (tensor.rs:228-250, ops/dropout.rs), tile
// (ops/pooling.rs:276-309), the fused residual + layernorm forward
// (ops/fused.rs:23-78) and gradient unscaling with its overflow check
// (ops/mixed_precision.rs:17-32).
#include "common.h"

// The reference's cpu arm rounds every multiply and every add separately (Rust
// never contracts a * b + c); these kernels are bandwidth-bound, so they do
// the same and stay as close to it as the summation order allows.
#pragma clang fp contract(off)

namespace mni {

static constexpr int TPB = 256;

static inline unsigned grid_for(int64_t n, int per_block) {
    int64_t b = (n + per_block - 1) / per_block;
    if (b < 1) b = 1;
    if (b > 0x7fffffffLL) b = 0x7fffffffLL;
    return (unsigned)b;
}
static __host__ __device__ inline bool al16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// ---- Philox4x32-10 ---------------------------------------------------------------
// Salmon et al., "Parallel random numbers: as easy as 1, 2, 3" (SC'11).  Element
// i of a stream uses word i % 4 of the block with counter (offset + i / 4) and
// the seed as key, so any element can be regenerated from (seed, offset, i):
// dropout's backward does that instead of storing a mask.
__device__ __forceinline__ uint4 philox4x32_10(uint64_t counter, uint64_t seed) {
    uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)(counter >> 32), c2 = 0u, c3 = 0u;
    uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        c0 = hi1 ^ c1 ^ k0;
        c1 = lo1;
        c2 = hi0 ^ c3 ^ k1;
        c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return make_uint4(c0, c1, c2, c3);
}
// 24 random bits -> [0, 1) in steps of 2^-24, the resolution of rand's f32
// sampling that the reference draws from.
__device__ __forceinline__ float u01(uint32_t w) { return (float)(w >> 8) * 5.9604644775390625e-8f; }
// Box-Muller on two words; the first uniform is shifted into (0, 1] so the
// logarithm is finite.
__device__ __forceinline__ void normal_pair(uint32_t w0, uint32_t w1, float *z0, float *z1) {
    const float u1 = (float)((w0 >> 8) + 1u) * 5.9604644775390625e-8f;
    const float u2 = u01(w1);
    const float r = sqrtf(-2.0f * logf(u1));
    const float a = 6.283185307179586f * u2;
    *z0 = r * cosf(a);
    *z1 = r * sinf(a);
}

// mode 0: uniform [0, 1); mode 1: standard normal; mode 2: raw words as floats' bit patterns (tests)
__global__ void random_fill_kernel(float *__restrict__ out, int64_t n, uint64_t seed, uint64_t offset, int mode) {
    int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    const int64_t nq = (n + 3) / 4;
    for (; q < nq; q += step) {
        const uint4 w = philox4x32_10(offset + (uint64_t)q, seed);
        float v[4];
        if (mode == 0) {
            v[0] = u01(w.x); v[1] = u01(w.y); v[2] = u01(w.z); v[3] = u01(w.w);
        } else if (mode == 1) {
            normal_pair(w.x, w.y, &v[0], &v[1]);
            normal_pair(w.z, w.w, &v[2], &v[3]);
        } else {
            v[0] = __uint_as_float(w.x); v[1] = __uint_as_float(w.y); v[2] = __uint_as_float(w.z); v[3] = __uint_as_float(w.w);
        }
        const int64_t base = q * 4;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (base + j < n) out[base + j] = v[j];
    }
}
int k_random_fill(float *out, int64_t n, uint64_t seed, uint64_t offset, int mode) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(random_fill_kernel, dim3(grid_for((n + 3) / 4, TPB * 2)), dim3(TPB), 0, ctx().stream, out, n, seed, offset,
                       mode);
    return check_launch("random_fill");
}

// ---- dropout (ops/dropout.rs:25-58, 114-126) --------------------------------------
// out = x * mask * scale with mask = (u >= rate), written out as the reference
// multiplies (so a dropped -3 gives -0 and a dropped inf gives NaN there too).
// The same kernel is the backward: pass the gradient as x.
__global__ void dropout_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t n, float rate, float scale,
                               uint64_t seed, uint64_t offset) {
    int64_t q = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    const int64_t nq = (n + 3) / 4;
    const bool vec = al16(out) && al16(x);
    for (; q < nq; q += step) {
        const uint4 w = philox4x32_10(offset + (uint64_t)q, seed);
        const float m[4] = {u01(w.x) >= rate ? 1.0f : 0.0f, u01(w.y) >= rate ? 1.0f : 0.0f, u01(w.z) >= rate ? 1.0f : 0.0f,
                            u01(w.w) >= rate ? 1.0f : 0.0f};
        const int64_t base = q * 4;
        if (vec && base + 4 <= n) {
            const float4 v = *reinterpret_cast<const float4 *>(x + base);
            *reinterpret_cast<float4 *>(out + base) =
                make_float4(v.x * m[0] * scale, v.y * m[1] * scale, v.z * m[2] * scale, v.w * m[3] * scale);
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                if (base + j < n) out[base + j] = x[base + j] * m[j] * scale;
        }
    }
}
int k_dropout(float *out, const float *x, int64_t n, float rate, float scale, uint64_t seed, uint64_t offset) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(dropout_kernel, dim3(grid_for((n + 3) / 4, TPB * 2)), dim3(TPB), 0, ctx().stream, out, x, n, rate, scale,
                       seed, offset);
    return check_launch("dropout");
}

// ---- dataset windows (ops/data.rs:79-155) -------------------------------------------
// inputs[b, t] = data[start_b + t], targets[b, t] = data[start_b + t + 1]
__global__ void sample_windows_kernel(int32_t *__restrict__ inputs, int32_t *__restrict__ targets,
                                      const int32_t *__restrict__ data, const int32_t *__restrict__ starts, int64_t block,
                                      int64_t total) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < total; i += step) {
        const int64_t b = i / block, t = i - b * block;
        const int64_t s = starts[b] + t;
        inputs[i] = data[s];
        targets[i] = data[s + 1];
    }
}
int k_sample_windows(int32_t *inputs, int32_t *targets, const int32_t *data, const int32_t *starts, int64_t block, int64_t batch) {
    const int64_t total = block * batch;
    if (total <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(sample_windows_kernel, dim3(grid_for(total, TPB)), dim3(TPB), 0, ctx().stream, inputs, targets, data,
                       starts, block, total);
    return check_launch("sample_windows");
}

// ---- embedding (ops/embedding.rs:25-53, 104-128) --------------------------------------
__global__ void embedding_gather4_kernel(float4 *__restrict__ out, const float4 *__restrict__ w,
                                         const int32_t *__restrict__ idx, int64_t dim4, int64_t total4) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < total4; i += step) {
        const int64_t tok = i / dim4, c = i - tok * dim4;
        out[i] = w[(int64_t)idx[tok] * dim4 + c];
    }
}
__global__ void embedding_gather_kernel(float *__restrict__ out, const float *__restrict__ w, const int32_t *__restrict__ idx,
                                        int64_t dim, int64_t total) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < total; i += step) {
        const int64_t tok = i / dim, c = i - tok * dim;
        out[i] = w[(int64_t)idx[tok] * dim + c];
    }
}
int k_embedding_forward(float *out, const float *w, const int32_t *idx, int64_t tokens, int64_t dim) {
    if (tokens <= 0 || dim <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if ((dim % 4) == 0 && al16(out) && al16(w))
        MNI_KERNEL_LAUNCH(embedding_gather4_kernel, dim3(grid_for(tokens * dim / 4, TPB * 2)), dim3(TPB), 0, ctx().stream,
                           reinterpret_cast<float4 *>(out), reinterpret_cast<const float4 *>(w), idx, dim / 4, tokens * dim / 4);
    else
        MNI_KERNEL_LAUNCH(embedding_gather_kernel, dim3(grid_for(tokens * dim, TPB * 2)), dim3(TPB), 0, ctx().stream, out, w,
                           idx, dim, tokens * dim);
    return check_launch("embedding_forward");
}

// The weight gradient dw[v, :] = sum over the tokens t with idx[t] == v of
// g[t, :], added in increasing t like the reference's loop, so the result does
// not depend on scheduling.  The tokens are bucketed by row with integer
// atomics (count, exclusive scan, unordered fill), every bucket is put in
// order by rank counting, and one workgroup per weight row then adds its
// bucket's gradient rows in that order (rows nobody used get zeros).
__global__ void emb_count_kernel(int32_t *__restrict__ count, const int32_t *__restrict__ idx, int64_t tokens) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; t < tokens; t += step) atomicAdd(&count[idx[t]], 1);
}
// start[0..vocab] = exclusive scan of count[0..vocab); one workgroup of 1024
__global__ void emb_scan_kernel(int32_t *__restrict__ start, const int32_t *__restrict__ count, int64_t vocab) {
    __shared__ int32_t part[1024];
    const int tid = threadIdx.x;
    const int64_t per = (vocab + 1023) / 1024;
    const int64_t lo = min(vocab, (int64_t)tid * per), hi = min(vocab, lo + per);
    int32_t s = 0;
    for (int64_t v = lo; v < hi; ++v) s += count[v];
    part[tid] = s;
    __syncthreads();
    for (int off = 1; off < 1024; off <<= 1) {
        const int32_t add = tid >= off ? part[tid - off] : 0;
        __syncthreads();
        part[tid] += add;
        __syncthreads();
    }
    int32_t run = part[tid] - s;  // exclusive prefix of this thread's chunk
    for (int64_t v = lo; v < hi; ++v) {
        start[v] = run;
        run += count[v];
    }
    if (tid == 1023) start[vocab] = part[1023];
}
__global__ void emb_fill_kernel(int32_t *__restrict__ list, int32_t *__restrict__ cursor, const int32_t *__restrict__ start,
                                const int32_t *__restrict__ idx, int64_t tokens) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; t < tokens; t += step) {
        const int32_t v = idx[t];
        list[start[v] + atomicAdd(&cursor[v], 1)] = (int32_t)t;
    }
}
__global__ void emb_order_kernel(int32_t *__restrict__ sorted, const int32_t *__restrict__ list,
                                 const int32_t *__restrict__ start, const int32_t *__restrict__ idx, int64_t tokens) {
    int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; t < tokens; t += step) {
        const int32_t v = idx[t];
        const int32_t s = start[v], e = start[v + 1];
        int32_t rank = 0;
        for (int32_t k = s; k < e; ++k) rank += list[k] < (int32_t)t ? 1 : 0;
        sorted[s + rank] = (int32_t)t;
    }
}
template <typename V>
__device__ __forceinline__ void emb_acc(V &a, const V &b);
template <>
__device__ __forceinline__ void emb_acc<float>(float &a, const float &b) { a += b; }
template <>
__device__ __forceinline__ void emb_acc<float4>(float4 &a, const float4 &b) { a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w; }
template <typename V>
__device__ __forceinline__ V emb_zero();
template <>
__device__ __forceinline__ float emb_zero<float>() { return 0.0f; }
template <>
__device__ __forceinline__ float4 emb_zero<float4>() { return make_float4(0.f, 0.f, 0.f, 0.f); }

template <typename V>
__global__ void emb_accumulate_kernel(V *__restrict__ dw, const V *__restrict__ g, const int32_t *__restrict__ sorted,
                                      const int32_t *__restrict__ start, int64_t dimv) {
    const int64_t v = blockIdx.x;
    const int32_t s = start[v], e = start[v + 1];
    for (int64_t c = (int64_t)blockIdx.y * blockDim.x + threadIdx.x; c < dimv; c += (int64_t)gridDim.y * blockDim.x) {
        V acc = emb_zero<V>();
        int32_t k = s;
        for (; k + 4 <= e; k += 4) {  // four gradient rows requested before the first add
            const int32_t t0 = sorted[k], t1 = sorted[k + 1], t2 = sorted[k + 2], t3 = sorted[k + 3];
            const V a0 = g[(int64_t)t0 * dimv + c], a1 = g[(int64_t)t1 * dimv + c];
            const V a2 = g[(int64_t)t2 * dimv + c], a3 = g[(int64_t)t3 * dimv + c];
            emb_acc(acc, a0); emb_acc(acc, a1); emb_acc(acc, a2); emb_acc(acc, a3);
        }
        for (; k < e; ++k) emb_acc(acc, g[(int64_t)sorted[k] * dimv + c]);
        dw[v * dimv + c] = acc;
    }
}
// `work` holds 3 * vocab + 2 + 2 * tokens int32 values
int k_embedding_backward(float *dw, const float *g, const int32_t *idx, int64_t tokens, int64_t vocab, int64_t dim,
                         int32_t *work) {
    if (vocab <= 0 || dim <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (vocab > 0x7fffffffLL || tokens > 0x7fffffffLL)
        return set_error(MNI_ERR_INVALID, "embedding backward: %lld rows / %lld tokens exceed the 32-bit index range",
                         (long long)vocab, (long long)tokens);
    int32_t *count = work, *cursor = work + vocab, *start = work + 2 * vocab, *list = start + vocab + 1 + 1,
            *sorted = list + tokens;
    // count and cursor start at zero (an all-zero bit pattern is 0 for both types)
    MNI_TRY(k_fill(reinterpret_cast<float *>(count), 0.0f, 2 * vocab));
    hipStream_t st = ctx().stream;
    if (tokens > 0) {
        MNI_KERNEL_LAUNCH(emb_count_kernel, dim3(grid_for(tokens, TPB)), dim3(TPB), 0, st, count, idx, tokens);
        MNI_TRY(check_launch("embedding_count"));
    }
    MNI_KERNEL_LAUNCH(emb_scan_kernel, dim3(1), dim3(1024), 0, st, start, (const int32_t *)count, vocab);
    MNI_TRY(check_launch("embedding_scan"));
    if (tokens > 0) {
        MNI_KERNEL_LAUNCH(emb_fill_kernel, dim3(grid_for(tokens, TPB)), dim3(TPB), 0, st, list, cursor, (const int32_t *)start,
                           idx, tokens);
        MNI_TRY(check_launch("embedding_fill"));
        MNI_KERNEL_LAUNCH(emb_order_kernel, dim3(grid_for(tokens, TPB)), dim3(TPB), 0, st, sorted, (const int32_t *)list,
                           (const int32_t *)start, idx, tokens);
        MNI_TRY(check_launch("embedding_order"));
    }
    if ((dim % 4) == 0 && al16(dw) && al16(g)) {
        const int64_t dimv = dim / 4;
        const int threads = dimv >= 256 ? 256 : dimv >= 128 ? 128 : 64;
        MNI_KERNEL_LAUNCH(emb_accumulate_kernel<float4>, dim3((unsigned)vocab, 1), dim3(threads), 0, st,
                           reinterpret_cast<float4 *>(dw), reinterpret_cast<const float4 *>(g), (const int32_t *)sorted,
                           (const int32_t *)start, dimv);
    } else {
        const int threads = dim >= 256 ? 256 : dim >= 128 ? 128 : 64;
        MNI_KERNEL_LAUNCH(emb_accumulate_kernel<float>, dim3((unsigned)vocab, 1), dim3(threads), 0, st, dw, g,
                           (const int32_t *)sorted, (const int32_t *)start, dim);
    }
    return check_launch("embedding_accumulate");
}

// ---- tile (ops/pooling.rs:276-309) ------------------------------------------------------
struct TileDesc {
    int ndim;
    int64_t in_shape[MNI_MAX_DIMS];
    int64_t in_strides[MNI_MAX_DIMS];
    int64_t out_strides[MNI_MAX_DIMS];
};
__global__ void tile_kernel(float *__restrict__ out, const float *__restrict__ in, const TileDesc d, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        int64_t rem = i, src = 0;
        for (int k = 0; k < d.ndim; ++k) {
            const int64_t coord = rem / d.out_strides[k];
            rem -= coord * d.out_strides[k];
            src += (coord % d.in_shape[k]) * d.in_strides[k];
        }
        out[i] = in[src];
    }
}
// `in` is contiguous over in_shape; out is contiguous over in_shape[k] * reps[k]
int k_tile(float *out, const float *in, const int64_t *in_shape, const int64_t *reps, int ndim) {
    if (ndim < 1 || ndim > MNI_MAX_DIMS) return set_error(MNI_ERR_INVALID, "tile: rank %d out of range", ndim);
    TileDesc d;
    d.ndim = ndim;
    int64_t n = 1, in_stride = 1, out_stride = 1;
    for (int k = ndim - 1; k >= 0; --k) {
        d.in_shape[k] = in_shape[k];
        d.in_strides[k] = in_stride;
        d.out_strides[k] = out_stride;
        in_stride *= in_shape[k];
        out_stride *= in_shape[k] * reps[k];
        n *= in_shape[k] * reps[k];
    }
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(tile_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, in, d, n);
    return check_launch("tile");
}

// ---- residual + layernorm forward (ops/fused.rs:23-78) -----------------------------------
// One wavefront per row: res = x + residual is stored (the backward needs it),
// then mean, biased variance over the centred values and the affine output.
__device__ __forceinline__ float seq_wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__global__ void residual_layernorm_kernel(float *__restrict__ out, float *__restrict__ res, float *__restrict__ mean,
                                          float *__restrict__ rstd, const float *__restrict__ x,
                                          const float *__restrict__ residual, const float *__restrict__ gamma,
                                          const float *__restrict__ beta, int64_t rows, int64_t c, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *px = x + row * c, *pr = residual + row * c;
    float *ps = res + row * c;
    float s = 0.f;
    for (int64_t j = lane; j < c; j += 64) {
        const float v = px[j] + pr[j];
        ps[j] = v;  // read back below by the lane that wrote it
        s += v;
    }
    const float m = seq_wave_sum(s) / (float)c;
    float var = 0.f;
    for (int64_t j = lane; j < c; j += 64) { const float d = ps[j] - m; var += d * d; }
    const float r = 1.0f / sqrtf(seq_wave_sum(var) / (float)c + eps);
    for (int64_t j = lane; j < c; j += 64) out[row * c + j] = (ps[j] - m) * r * gamma[j] + beta[j];
    if (lane == 0) { mean[row] = m; rstd[row] = r; }
}
int k_residual_layernorm(float *out, float *res, float *mean, float *rstd, const float *x, const float *residual,
                         const float *gamma, const float *beta, int64_t rows, int64_t c, float eps) {
    if (rows <= 0 || c <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (launch_layernorm_workgroups(out, res, mean, rstd, x, residual, gamma, beta, rows, c, eps)) return check_launch("residual_layernorm");
    MNI_KERNEL_LAUNCH(residual_layernorm_kernel, dim3(grid_for(rows, 4)), dim3(TPB), 0, ctx().stream, out, res, mean, rstd, x,
                       residual, gamma, beta, rows, c, eps);
    return check_launch("residual_layernorm");
}

// ---- gradient unscale + overflow check (ops/mixed_precision.rs:17-32) ----------------------
// g *= s; *flag = 1 when any scaled value is infinite or NaN (every writer
// stores the same value, so the race between them is harmless).
__global__ void scale_check_kernel(float *__restrict__ g, float s, int64_t n, float *__restrict__ flag) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    bool bad = false;
    for (; i < n; i += step) {
        const float v = g[i] * s;
        g[i] = v;
        bad |= !(fabsf(v) <= 3.402823466e+38f);
    }
    if (bad) *flag = 1.0f;
}
int k_scale_check(float *g, float s, int64_t n, float *flag) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(scale_check_kernel, dim3(grid_for(n, TPB * 4)), dim3(TPB), 0, ctx().stream, g, s, n, flag);
    return check_launch("scale_check");
}

}  // namespace mni
