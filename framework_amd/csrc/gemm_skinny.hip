// Skinny (GEMV-shaped) fp32 products for gfx950: a few rows of X against a
// large W.  These are bound by streaming W once from HBM, so they use plain
// FMAs, 16-byte loads with many loads in flight per lane, and wavefront / LDS
// reductions -- no MFMA.  The reference has no such special case: its cuda arm
// sends every shape to cuBLAS (src/native/src/ops/matmul.rs:150-189).
#include "common.h"
#include "gemm_internal.h"

namespace mni {

static constexpr int SK_THREADS = 256;   // skinny_cols: 4 wavefronts per workgroup
static constexpr int SK_WAVES = SK_THREADS / 64;
static constexpr int SK_COLS = 256;      // columns per workgroup: 64 lanes x float4
static constexpr int SK_UNROLL = 16;     // W rows in flight per lane
typedef float f32x4 __attribute__((ext_vector_type(4)));

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
// grid = (column groups of 256, K slices, batch), 256 threads = 4 wavefronts.
// A wavefront reads whole 1 KiB pieces of W rows (every lane one 16-byte load
// per row, SK_UNROLL rows in flight), which is the access pattern that streams
// HBM best; the X values of a row are the same for all lanes, so they are
// fetched with wave-uniform (scalar) loads.  The 4 wavefronts interleave groups
// of SK_UNROLL rows and are summed through LDS in wave order.  K is sliced
// across workgroups until about 4 workgroups per CU exist; each slice leaves a
// partial that skinny_reduce_kernel sums in slice order, so the result does not
// depend on scheduling.  (Single-launch variants -- arrival counters with
// device-scope fences, float atomics, write-through partial stores, or one
// workgroup owning all of K for 16 columns -- were measured slower on MI355X:
// cross-XCD communication inside a kernel costs more than a second launch.)
template <int MR, bool XC>
__global__ __launch_bounds__(SK_THREADS) void skinny_cols_kernel(const SkinnyLaunch s) {
    constexpr int U = SK_UNROLL;
    __shared__ float4 red[SK_WAVES - 1][MR][64];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int col0 = blockIdx.x * SK_COLS + 4 * lane;
    const int slice = blockIdx.y, b = blockIdx.z;
    const int k_begin = slice * s.k_per_slice;
    const int k_end = min(s.K, k_begin + s.k_per_slice);
    const bool col_ok = col0 < s.cols;  // cols % 4 == 0 is a launch precondition

    const float *__restrict__ X = s.X + (int64_t)(b % s.x_bcount) * s.x_bs;
    const float *__restrict__ W = s.W + (int64_t)(b % s.w_bcount) * s.w_bs + (col_ok ? col0 : 0);

    float4 acc[MR];
#pragma unroll
    for (int i = 0; i < MR; ++i) acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);

    for (int k0 = k_begin + wave * U; k0 < k_end; k0 += SK_WAVES * U) {
        f32x4 w[U];
        if (k0 + U <= k_end) {
            // whole group inside the slice: no clamps, no guards
            const float *__restrict__ wp = W + (int64_t)k0 * s.w_rs;
#pragma unroll
            for (int u = 0; u < U; ++u)
                w[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(wp + (int64_t)u * s.w_rs));
#pragma unroll
            for (int i = 0; i < MR; ++i) {
                if (i < s.rows) {
                    float xv[U];
                    if (XC) {  // X rows contiguous along k: one scalar load of U floats
                        const float *__restrict__ xr = X + (int64_t)i * s.x_rs + k0;
#pragma unroll
                        for (int u = 0; u < U; ++u) xv[u] = xr[u];
                    } else {
                        const float *__restrict__ xr = X + (int64_t)i * s.x_rs + (int64_t)k0 * s.x_cs;
#pragma unroll
                        for (int u = 0; u < U; ++u) xv[u] = xr[(int64_t)u * s.x_cs];
                    }
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        acc[i].x += xv[u] * w[u].x;
                        acc[i].y += xv[u] * w[u].y;
                        acc[i].z += xv[u] * w[u].z;
                        acc[i].w += xv[u] * w[u].w;
                    }
                }
            }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                // rows past the slice re-read its last row and meet x == 0
                const int krow = min(k0 + u, k_end - 1);
                w[u] = *reinterpret_cast<const f32x4 *>(W + (int64_t)krow * s.w_rs);
            }
#pragma unroll
            for (int i = 0; i < MR; ++i) {
                if (i < s.rows) {
                    const float *__restrict__ xr = X + (int64_t)i * s.x_rs + (int64_t)k0 * s.x_cs;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const float xv = (k0 + u < k_end) ? xr[(int64_t)u * s.x_cs] : 0.0f;
                        acc[i].x += xv * w[u].x;
                        acc[i].y += xv * w[u].y;
                        acc[i].z += xv * w[u].z;
                        acc[i].w += xv * w[u].w;
                    }
                }
            }
        }
    }

    // ---- sum the wavefronts in wave order -------------------------------------
    if (wave > 0) {
#pragma unroll
        for (int i = 0; i < MR; ++i) red[wave - 1][i][lane] = acc[i];
    }
    __syncthreads();
    if (wave != 0 || !col_ok) return;
#pragma unroll
    for (int i = 0; i < MR; ++i) {
#pragma unroll
        for (int w = 0; w < SK_WAVES - 1; ++w) {
            const float4 p = red[w][i][lane];
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
        if (i < s.rows) {
            float r[4] = {acc[i].x, acc[i].y, acc[i].z, acc[i].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (s.epilogue != MNI_EPI_NONE) r[e] = sk_epilogue(r[e], s.bias[s.bias_on_rows ? i : col0 + e], s.epilogue);
                float *dst = out + (int64_t)i * s.o_rs + (int64_t)(col0 + e) * s.o_cs;
                *dst = s.accumulate ? r[e] + *dst : r[e];
            }
        }
    }
}

// Sums the K-slice partials ws[slice][batch][rows][cols] of a skinny product.
// The outputs are few and the slices many, so a workgroup of 16 wavefronts
// takes 64 outputs and spreads the slices over its wavefronts (wavefront g adds
// slices g, g + 16, ... in order, up to 4 loads in flight); the 16 sums are then
// combined in wavefront order.  The grouping depends only on the slice count,
// so the result is reproducible.
static constexpr int RED_GROUPS = 16;
__global__ __launch_bounds__(64 * RED_GROUPS) void skinny_reduce_kernel(const ReduceLaunch r) {
    __shared__ float sh[RED_GROUPS][64];
    const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int64_t per_batch = (int64_t)r.rows * r.cols;
    const int64_t total = per_batch * r.batch;
    const int64_t idx = (int64_t)blockIdx.x * 64 + lane;
    float t = 0.0f;
    if (idx < total) {
        const float *p = r.ws + idx;
        int sl = g;
        for (; sl + 3 * RED_GROUPS < r.slices; sl += 4 * RED_GROUPS) {
            const float a = p[(int64_t)sl * total], b = p[(int64_t)(sl + RED_GROUPS) * total];
            const float c = p[(int64_t)(sl + 2 * RED_GROUPS) * total], d = p[(int64_t)(sl + 3 * RED_GROUPS) * total];
            t += a; t += b; t += c; t += d;
        }
        for (; sl < r.slices; sl += RED_GROUPS) t += p[(int64_t)sl * total];
    }
    sh[g][lane] = t;
    __syncthreads();
    if (g != 0 || idx >= total) return;
    float v = sh[0][lane];
#pragma unroll
    for (int k = 1; k < RED_GROUPS; ++k) v += sh[k][lane];
    const int b = (int)(idx / per_batch);
    const int64_t rem = idx - (int64_t)b * per_batch;
    const int i = (int)(rem / r.cols), j = (int)(rem - (int64_t)i * r.cols);
    if (r.epilogue != MNI_EPI_NONE) v = sk_epilogue(v, r.bias[r.bias_on_rows ? i : j], r.epilogue);
    float *dst = r.out + (int64_t)b * r.o_bs + (int64_t)i * r.o_rs + (int64_t)j * r.o_cs;
    if (r.accumulate) v += *dst;
    *dst = v;
}

// ---- W contiguous along K ------------------------------------------------------
// One wavefront per 4 output columns: lanes stride K with 16-byte loads of X
// and of the 4 W columns, then a butterfly reduction across the wavefront.
template <int MR>
__global__ __launch_bounds__(256) void skinny_dots_kernel(const SkinnyLaunch s) {
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
int skinny_cols_rows_per_pass() { return SK_WAVES * SK_UNROLL; }

int launch_skinny_cols(const SkinnyLaunch &s) {
    if (s.rows <= 0 || s.cols <= 0 || s.batch <= 0) return MNI_OK;
    dim3 grid((s.cols + SK_COLS - 1) / SK_COLS, s.split_k, s.batch), block(SK_THREADS);
    hipStream_t st = ctx().stream;
    const bool xc = s.x_cs == 1;
#define MNI_SK(MR)                                                                          \
    do {                                                                                    \
        if (xc) hipLaunchKernelGGL((skinny_cols_kernel<MR, true>), grid, block, 0, st, s);  \
        else hipLaunchKernelGGL((skinny_cols_kernel<MR, false>), grid, block, 0, st, s);    \
    } while (0)
    if (s.rows <= 4) MNI_SK(4);
    else if (s.rows <= 8) MNI_SK(8);
    else if (s.rows <= 16) MNI_SK(16);
    else return set_error(MNI_ERR_INVALID, "skinny kernel takes at most 16 rows, got %d", s.rows);
#undef MNI_SK
    return check_launch("skinny_cols_kernel");
}

int launch_skinny_reduce(const ReduceLaunch &r) {
    const int64_t total = (int64_t)r.rows * r.cols * r.batch;
    if (total <= 0) return MNI_OK;
    hipLaunchKernelGGL(skinny_reduce_kernel, dim3((unsigned)((total + 63) / 64)), dim3(64 * RED_GROUPS), 0, ctx().stream, r);
    return check_launch("skinny_reduce_kernel");
}

int launch_skinny_dots(const SkinnyLaunch &s) {
    if (s.rows <= 0 || s.cols <= 0 || s.batch <= 0) return MNI_OK;
    dim3 grid((s.cols + 15) / 16, s.batch), block(256);
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
