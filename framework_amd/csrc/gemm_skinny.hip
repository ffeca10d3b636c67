// Skinny (GEMV-shaped) fp32 products for gfx950: a few rows of X against a
// large W.  These are bound by streaming W once from HBM, so they use plain
// FMAs, 16-byte loads with many loads in flight per lane, and wavefront / LDS
// reductions -- no MFMA.  The reference has no such special case: its cuda arm
// sends every shape to cuBLAS (src/native/src/ops/matmul.rs:150-189).
#include "common.h"
#include "gemm_internal.h"

namespace mni {

static constexpr int SK_THREADS = 256;
static constexpr int SK_COLS = 256;    // columns per workgroup: 64 lanes x float4
static constexpr int SK_KCHUNK = 256;  // K rows of X staged in LDS at a time
static constexpr int SK_UNROLL = 8;    // W rows in flight per lane

__device__ __forceinline__ float sk_gelu(float x) {
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}

__device__ __forceinline__ float sk_epilogue(float v, float bias, int epilogue) {
    v += bias;
    if (epilogue == MNI_EPI_BIAS_RELU) v = fmaxf(v, 0.0f);
    else if (epilogue == MNI_EPI_BIAS_GELU) v = sk_gelu(v);
    return v;
}

// ---- W contiguous along columns ---------------------------------------------
// grid = (column groups, K slices, batch).  Every lane owns 4 consecutive
// columns; the 4 wavefronts of a workgroup take interleaved groups of 8 K rows
// and are summed through LDS in wave order, so the result is deterministic.
template <int MR>
__global__ __launch_bounds__(SK_THREADS) void skinny_cols_kernel(const SkinnyLaunch s) {
    // One buffer, two lives: X staging during the K loop, wave partials after.
    __shared__ float smem[3 * 16 * SK_COLS];  // 48 KB
    float(*xs)[SK_KCHUNK] = reinterpret_cast<float(*)[SK_KCHUNK]>(smem);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int col0 = blockIdx.x * SK_COLS + 4 * lane;
    const int slice = blockIdx.y, b = blockIdx.z;
    const int k_begin = slice * s.k_per_slice;
    const int k_end = min(s.K, k_begin + s.k_per_slice);
    const bool col_ok = col0 < s.cols;  // cols % 4 == 0 is a launch precondition

    const float *__restrict__ X = s.X + (int64_t)(b % s.x_bcount) * s.x_bs;
    const float *__restrict__ W = s.W + (int64_t)(b % s.w_bcount) * s.w_bs + col0;

    float4 acc[MR];
#pragma unroll
    for (int i = 0; i < MR; ++i) acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);

    for (int kc = k_begin; kc < k_end; kc += SK_KCHUNK) {
        const int kn = min(SK_KCHUNK, k_end - kc);
        __syncthreads();
        for (int idx = tid; idx < MR * SK_KCHUNK; idx += SK_THREADS) {
            const int i = idx / SK_KCHUNK, kk = idx - i * SK_KCHUNK;
            xs[i][kk] = (i < s.rows && kk < kn) ? X[(int64_t)i * s.x_rs + (int64_t)(kc + kk) * s.x_cs] : 0.0f;
        }
        __syncthreads();
        if (col_ok) {
            for (int kk = wave * SK_UNROLL; kk < kn; kk += 4 * SK_UNROLL) {
                float4 w[SK_UNROLL];
#pragma unroll
                for (int u = 0; u < SK_UNROLL; ++u) {
                    // rows past the chunk read row kk (in range) and meet x == 0
                    const int krow = kc + (kk + u < kn ? kk + u : kk);
                    w[u] = *reinterpret_cast<const float4 *>(W + (int64_t)krow * s.w_rs);
                }
#pragma unroll
                for (int i = 0; i < MR; ++i) {
                    const float4 x0 = *reinterpret_cast<const float4 *>(&xs[i][kk]);
                    const float4 x1 = *reinterpret_cast<const float4 *>(&xs[i][kk + 4]);
                    const float xv[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
#pragma unroll
                    for (int u = 0; u < SK_UNROLL; ++u) {
                        acc[i].x += xv[u] * w[u].x;
                        acc[i].y += xv[u] * w[u].y;
                        acc[i].z += xv[u] * w[u].z;
                        acc[i].w += xv[u] * w[u].w;
                    }
                }
            }
        }
    }

    // ---- sum the 4 wavefronts in wave order ---------------------------------
    __syncthreads();
    float4 *red = reinterpret_cast<float4 *>(smem);  // [3][MR][64]
    if (wave > 0) {
#pragma unroll
        for (int i = 0; i < MR; ++i) red[((wave - 1) * MR + i) * 64 + lane] = acc[i];
    }
    __syncthreads();
    if (wave != 0 || !col_ok) return;
#pragma unroll
    for (int i = 0; i < MR; ++i) {
#pragma unroll
        for (int w = 0; w < 3; ++w) {
            const float4 p = red[(w * MR + i) * 64 + lane];
            acc[i].x += p.x; acc[i].y += p.y; acc[i].z += p.z; acc[i].w += p.w;
        }
    }

    if (s.split_k > 1) {
        float *ws = s.ws + (((int64_t)slice * s.batch + b) * s.rows) * (int64_t)s.cols + col0;
#pragma unroll
        for (int i = 0; i < MR; ++i)
            if (i < s.rows) *reinterpret_cast<float4 *>(ws + (int64_t)i * s.cols) = acc[i];
        return;
    }
    float *out = s.out + (int64_t)b * s.o_bs;
#pragma unroll
    for (int i = 0; i < MR; ++i) {
        if (i >= s.rows) break;
        float v[4] = {acc[i].x, acc[i].y, acc[i].z, acc[i].w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float *dst = out + (int64_t)i * s.o_rs + (int64_t)(col0 + e) * s.o_cs;
            float r = v[e];
            if (s.epilogue != MNI_EPI_NONE) r = sk_epilogue(r, s.bias[s.bias_on_rows ? i : col0 + e], s.epilogue);
            if (s.accumulate) r += *dst;
            *dst = r;
        }
    }
}

// ---- W contiguous along K ------------------------------------------------------
// One wavefront per 4 output columns: lanes stride K with 16-byte loads of X
// and of the 4 W columns, then a butterfly reduction across the wavefront.
template <int MR>
__global__ __launch_bounds__(SK_THREADS) void skinny_dots_kernel(const SkinnyLaunch s) {
    constexpr int JW = 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j0 = (blockIdx.x * 4 + wave) * JW;
    const int b = blockIdx.y;
    if (j0 >= s.cols) return;

    const float *__restrict__ X = s.X + (int64_t)(b % s.x_bcount) * s.x_bs;
    const float *__restrict__ W = s.W + (int64_t)(b % s.w_bcount) * s.w_bs;
    const float *wp[JW];
#pragma unroll
    for (int c = 0; c < JW; ++c) wp[c] = W + (int64_t)min(j0 + c, s.cols - 1) * s.w_cs;

    float acc[MR][JW];
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int c = 0; c < JW; ++c) acc[i][c] = 0.0f;

    for (int k = 4 * lane; k < s.K; k += 256) {  // K % 4 == 0 is a launch precondition
        float4 w[JW];
#pragma unroll
        for (int c = 0; c < JW; ++c) w[c] = *reinterpret_cast<const float4 *>(wp[c] + k);
#pragma unroll
        for (int i = 0; i < MR; ++i) {
            const int ii = i < s.rows ? i : 0;
            const float4 x = *reinterpret_cast<const float4 *>(X + (int64_t)ii * s.x_rs + k);
#pragma unroll
            for (int c = 0; c < JW; ++c)
                acc[i][c] += x.x * w[c].x + x.y * w[c].y + x.z * w[c].z + x.w * w[c].w;
        }
    }
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int c = 0; c < JW; ++c) {
            float v = acc[i][c];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
            acc[i][c] = v;
        }
    if (lane != 0) return;
    float *out = s.out + (int64_t)b * s.o_bs;
#pragma unroll
    for (int i = 0; i < MR; ++i) {
        if (i >= s.rows) break;
#pragma unroll
        for (int c = 0; c < JW; ++c) {
            const int j = j0 + c;
            if (j >= s.cols) break;
            float *dst = out + (int64_t)i * s.o_rs + (int64_t)j * s.o_cs;
            float r = acc[i][c];
            if (s.epilogue != MNI_EPI_NONE) r = sk_epilogue(r, s.bias[s.bias_on_rows ? i : j], s.epilogue);
            if (s.accumulate) r += *dst;
            *dst = r;
        }
    }
}

// ---- split-K reduction ---------------------------------------------------------
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const ReduceLaunch r) {
    const int64_t per_batch = (int64_t)r.rows * r.cols;
    const int64_t total = per_batch * r.batch;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    float v = 0.0f;
    for (int sl = 0; sl < r.slices; ++sl) v += r.ws[(int64_t)sl * total + idx];
    const int b = (int)(idx / per_batch);
    const int64_t rem = idx - (int64_t)b * per_batch;
    const int i = (int)(rem / r.cols), j = (int)(rem - (int64_t)i * r.cols);
    if (r.epilogue != MNI_EPI_NONE) v = sk_epilogue(v, r.bias[r.bias_on_rows ? i : j], r.epilogue);
    float *dst = r.out + (int64_t)b * r.o_bs + (int64_t)i * r.o_rs + (int64_t)j * r.o_cs;
    if (r.accumulate) v += *dst;
    *dst = v;
}

int skinny_cols_block_cols() { return SK_COLS; }

int launch_skinny_cols(const SkinnyLaunch &s) {
    if (s.rows <= 0 || s.cols <= 0 || s.batch <= 0) return MNI_OK;
    dim3 grid((s.cols + SK_COLS - 1) / SK_COLS, s.split_k, s.batch), block(SK_THREADS);
    hipStream_t st = ctx().stream;
    if (s.rows <= 4) hipLaunchKernelGGL((skinny_cols_kernel<4>), grid, block, 0, st, s);
    else if (s.rows <= 8) hipLaunchKernelGGL((skinny_cols_kernel<8>), grid, block, 0, st, s);
    else if (s.rows <= 16) hipLaunchKernelGGL((skinny_cols_kernel<16>), grid, block, 0, st, s);
    else return set_error(MNI_ERR_INVALID, "skinny kernel takes at most 16 rows, got %d", s.rows);
    return check_launch("skinny_cols_kernel");
}

int launch_skinny_dots(const SkinnyLaunch &s) {
    if (s.rows <= 0 || s.cols <= 0 || s.batch <= 0) return MNI_OK;
    dim3 grid((s.cols + 15) / 16, s.batch), block(SK_THREADS);
    hipStream_t st = ctx().stream;
    if (s.rows <= 4) hipLaunchKernelGGL((skinny_dots_kernel<4>), grid, block, 0, st, s);
    else if (s.rows <= 8) hipLaunchKernelGGL((skinny_dots_kernel<8>), grid, block, 0, st, s);
    else if (s.rows <= 16) hipLaunchKernelGGL((skinny_dots_kernel<16>), grid, block, 0, st, s);
    else return set_error(MNI_ERR_INVALID, "skinny kernel takes at most 16 rows, got %d", s.rows);
    return check_launch("skinny_dots_kernel");
}

int launch_splitk_reduce(const ReduceLaunch &r) {
    const int64_t total = (int64_t)r.rows * r.cols * r.batch;
    if (total <= 0) return MNI_OK;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    hipLaunchKernelGGL(splitk_reduce_kernel, grid, block, 0, ctx().stream, r);
    return check_launch("splitk_reduce_kernel");
}

}  // namespace mni
