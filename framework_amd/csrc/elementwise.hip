// Bandwidth-bound support kernels around the GEMM path: fills, copies,
// strided gathers (views made contiguous on the device), broadcast binary ops,
// the Linear bias add and its column-sum gradient, activations, reductions
// along one dim, cross-entropy and the AdamW update.  They replace the
// per-element host loops of the reference's cpu arm (file:line at each kernel)
// and the 256-thread one-element-per-thread kernels of its cuda arm
// (src/native/kernels/elementwise.cu) with 16-byte accesses where the layout
// allows.
#include <string.h>

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
static inline bool al16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

__device__ __forceinline__ float d_gelu(float x) {
    // src/native/src/ops/activation.rs:15-18
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}
__device__ __forceinline__ float d_gelu_grad(float x) {
    // src/native/src/ops/activation.rs:20-28
    const float s = 0.7978845608028654f;
    const float inner = s * (x + 0.044715f * x * x * x);
    const float th = tanhf(inner);
    const float sech2 = 1.0f - th * th;
    const float d_inner = s * (1.0f + 3.0f * 0.044715f * x * x);
    return 0.5f * (1.0f + th) + 0.5f * x * sech2 * d_inner;
}

// ---- fill / axpy / scale ------------------------------------------------------
__global__ void fill_kernel(float *__restrict__ dst, float v, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = v;
}
__global__ void fill4_kernel(float4 *__restrict__ dst, float v, int64_t n4) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    const float4 f = make_float4(v, v, v, v);
    for (; i < n4; i += stride) dst[i] = f;
}
int k_fill(float *dst, float v, int64_t n) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (al16(dst) && (n % 4) == 0) {
        MNI_KERNEL_LAUNCH(fill4_kernel, dim3(grid_for(n / 4, TPB * 4)), dim3(TPB), 0, ctx().stream,
                           reinterpret_cast<float4 *>(dst), v, n / 4);
    } else {
        MNI_KERNEL_LAUNCH(fill_kernel, dim3(grid_for(n, TPB * 4)), dim3(TPB), 0, ctx().stream, dst, v, n);
    }
    return check_launch("fill");
}

// dst += alpha * src  (src/native/src/tensor.rs:272-290 accumulate_grad / add_inplace)
__global__ void axpy_kernel(float *__restrict__ dst, const float *__restrict__ src, float alpha, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] += alpha * src[i];
}
__global__ void axpy4_kernel(float4 *__restrict__ dst, const float4 *__restrict__ src, float alpha, int64_t n4) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n4; i += stride) {
        float4 d = dst[i];
        const float4 s = src[i];
        d.x += alpha * s.x; d.y += alpha * s.y; d.z += alpha * s.z; d.w += alpha * s.w;
        dst[i] = d;
    }
}
int k_axpy(float *dst, const float *src, float alpha, int64_t n) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (al16(dst) && al16(src) && (n % 4) == 0) {
        MNI_KERNEL_LAUNCH(axpy4_kernel, dim3(grid_for(n / 4, TPB * 2)), dim3(TPB), 0, ctx().stream,
                           reinterpret_cast<float4 *>(dst), reinterpret_cast<const float4 *>(src), alpha, n / 4);
    } else {
        MNI_KERNEL_LAUNCH(axpy_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, dst, src, alpha, n);
    }
    return check_launch("axpy");
}

__global__ void scale_kernel(float *__restrict__ dst, float s, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] *= s;
}
int k_scale_inplace(float *dst, float s, int64_t n) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(scale_kernel, dim3(grid_for(n, TPB * 4)), dim3(TPB), 0, ctx().stream, dst, s, n);
    return check_launch("scale");
}

// ---- strided gather -------------------------------------------------------------
// dst[i] = src[sum_d coord_d(i) * stride_d]: make_contiguous_data
// (src/native/src/tensor.rs:292-309) and permute_f32
// (src/native/kernels/elementwise.cu:67-81) without the 4-dim / i32 limits.
struct GatherDesc {
    int ndim;
    int64_t shape[MNI_MAX_DIMS];
    int64_t strides[MNI_MAX_DIMS];
};
__global__ void gather_kernel(float *__restrict__ dst, const float *__restrict__ src, const GatherDesc d, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        int64_t rem = i, off = 0;
        for (int k = d.ndim - 1; k >= 0; --k) {
            const int64_t c = rem % d.shape[k];
            rem /= d.shape[k];
            off += c * d.strides[k];
        }
        dst[i] = src[off];
    }
}
// The same when the innermost dim has unit stride in the source and a length
// that is a multiple of 4, with 16-byte aligned pieces (heads split off and
// merged back, [b, t, h, d] <-> [b, h, t, d]): one 16-byte access per four
// elements and a quarter of the index arithmetic.  d.shape / d.strides describe
// the dims above the innermost one; inner4 = innermost length / 4.
__global__ void gather4_kernel(float4 *__restrict__ dst, const float *__restrict__ src, const GatherDesc d, int64_t inner4,
                               int64_t n4) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n4; i += step) {
        int64_t rem = i / inner4;
        int64_t off = (i - rem * inner4) * 4;
        for (int k = d.ndim - 1; k >= 0; --k) {
            const int64_t c = rem % d.shape[k];
            rem /= d.shape[k];
            off += c * d.strides[k];
        }
        dst[i] = *reinterpret_cast<const float4 *>(src + off);
    }
}
// Batched 2-D transpose through LDS for the common "swap the last two dims"
// view: src element (b, r, c) at b*bs + r*1 + c*cs_ (row axis contiguous in
// memory), dst contiguous [b][r][c].
__global__ void transpose_tile_kernel(float *__restrict__ dst, const float *__restrict__ src, int64_t rows,
                                      int64_t cols, int64_t src_col_stride, int64_t src_bs) {
    __shared__ float tile[32][33];
    const int64_t b = blockIdx.z;
    const int64_t r0 = (int64_t)blockIdx.y * 32, c0 = (int64_t)blockIdx.x * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    const float *s = src + b * src_bs;
    float *d = dst + b * rows * cols;
    for (int j = ty; j < 32; j += 8) {
        const int64_t r = r0 + tx, c = c0 + j;  // read along r (contiguous)
        if (r < rows && c < cols) tile[j][tx] = s[r + c * src_col_stride];
    }
    __syncthreads();
    for (int j = ty; j < 32; j += 8) {
        const int64_t r = r0 + j, c = c0 + tx;  // write along c (contiguous)
        if (r < rows && c < cols) d[r * cols + c] = tile[tx][j];
    }
}
int k_strided_copy(float *dst, const float *src, const int64_t *shape, const int64_t *strides, int ndim) {
    MNI_TRY(ensure_init());
    if (ndim < 0 || ndim > MNI_MAX_DIMS) return set_error(MNI_ERR_INVALID, "strided_copy: ndim %d out of range", ndim);
    int64_t n = 1;
    for (int i = 0; i < ndim; ++i) {
        if (shape[i] < 0) return set_error(MNI_ERR_INVALID, "strided_copy: negative extent");
        n *= shape[i];
    }
    if (n == 0) return MNI_OK;
    // Fast path: last two dims swapped relative to memory, leading dims with
    // one uniform stride.
    if (ndim >= 2 && strides[ndim - 2] == 1 && shape[ndim - 2] > 1 && shape[ndim - 1] > 1) {
        const int64_t rows = shape[ndim - 2], cols = shape[ndim - 1];
        int64_t batch = 1, bs = 0;
        bool uniform = true;
        if (ndim > 2) {
            bs = strides[ndim - 3];
            int64_t expect = bs;
            for (int k = ndim - 3; k >= 0; --k) {
                if (shape[k] != 1 && strides[k] != expect) uniform = false;
                expect *= shape[k];
                batch *= shape[k];
            }
        }
        if (uniform && batch <= 65535) {
            dim3 grid((unsigned)((cols + 31) / 32), (unsigned)((rows + 31) / 32), (unsigned)batch);
            if (grid.y <= 65535) {
                MNI_KERNEL_LAUNCH(transpose_tile_kernel, grid, dim3(256), 0, ctx().stream, dst, src, rows, cols,
                                   strides[ndim - 1], bs);
                return check_launch("transpose_tile");
            }
        }
    }
    GatherDesc d;
    if (ndim >= 1 && strides[ndim - 1] == 1 && (shape[ndim - 1] % 4) == 0 && al16(dst) && al16(src)) {
        bool aligned = true;
        for (int i = 0; i < ndim - 1; ++i) aligned = aligned && (strides[i] % 4) == 0;
        if (aligned) {
            d.ndim = ndim - 1;
            for (int i = 0; i < ndim - 1; ++i) { d.shape[i] = shape[i]; d.strides[i] = strides[i]; }
            MNI_KERNEL_LAUNCH(gather4_kernel, dim3(grid_for(n / 4, TPB * 2)), dim3(TPB), 0, ctx().stream,
                               reinterpret_cast<float4 *>(dst), src, d, shape[ndim - 1] / 4, n / 4);
            return check_launch("gather4");
        }
    }
    d.ndim = ndim;
    for (int i = 0; i < ndim; ++i) { d.shape[i] = shape[i]; d.strides[i] = strides[i]; }
    MNI_KERNEL_LAUNCH(gather_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, dst, src, d, n);
    return check_launch("gather");
}

// ---- broadcast binary -----------------------------------------------------------
// broadcast_binary (src/native/src/ops/elementwise.rs:20-56): operands are
// addressed by their own strides with 0 on broadcast dims, so views need no copy.
__device__ __forceinline__ float bin_apply(float x, float y, int op, float p) {
    switch (op) {
    case BIN_ADD: return x + y;
    case BIN_SUB: return x - y;
    case BIN_MUL: return x * y;
    case BIN_DIV: return x / y;                               // elementwise.rs:918-928
    case BIN_LT: return x < y ? 1.0f : 0.0f;                  // :1099-1103
    case BIN_EQ: return x == y ? 1.0f : 0.0f;                 // :1152-1156
    case BIN_GT: return x > y ? 1.0f : 0.0f;                  // :1205-1209
    default: return fabsf(x - y) < p ? 1.0f : 0.0f;           // is_close, :1258-1288
    }
}
__global__ void binary_bcast_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ b,
                                    const StridedDesc d, int64_t n, int op, float p) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        int64_t rem = i, ao = 0, bo = 0;
        for (int k = d.ndim - 1; k >= 0; --k) {
            const int64_t c = rem % d.shape[k];
            rem /= d.shape[k];
            ao += c * d.a_strides[k];
            bo += c * d.b_strides[k];
        }
        out[i] = bin_apply(a[ao], b[bo], op, p);
    }
}
int k_binary_broadcast(float *out, const float *a, const float *b, const StridedDesc &d, int op, float p) {
    MNI_TRY(ensure_init());
    int64_t n = 1;
    for (int i = 0; i < d.ndim; ++i) n *= d.shape[i];
    if (n <= 0) return MNI_OK;
    MNI_KERNEL_LAUNCH(binary_bcast_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, a, b, d, n, op, p);
    return check_launch("binary_broadcast");
}

__global__ void binary_same_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ b,
                                   int64_t n, int op, float p) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) out[i] = bin_apply(a[i], b[i], op, p);
}
__global__ void binary_same4_kernel(float4 *__restrict__ out, const float4 *__restrict__ a,
                                    const float4 *__restrict__ b, int64_t n4, int op, float p) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n4; i += step) {
        const float4 x = a[i], y = b[i];
        out[i] = make_float4(bin_apply(x.x, y.x, op, p), bin_apply(x.y, y.y, op, p), bin_apply(x.z, y.z, op, p),
                             bin_apply(x.w, y.w, op, p));
    }
}
int k_binary_same(float *out, const float *a, const float *b, int64_t n, int op, float p) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (al16(out) && al16(a) && al16(b) && (n % 4) == 0) {
        MNI_KERNEL_LAUNCH(binary_same4_kernel, dim3(grid_for(n / 4, TPB * 2)), dim3(TPB), 0, ctx().stream,
                           reinterpret_cast<float4 *>(out), reinterpret_cast<const float4 *>(a),
                           reinterpret_cast<const float4 *>(b), n / 4, op, p);
    } else {
        MNI_KERNEL_LAUNCH(binary_same_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, a, b, n, op, p);
    }
    return check_launch("binary_same");
}

// div_backward (src/native/src/ops/elementwise.rs:991-1029) before the unbroadcast
__global__ void div_bwd_kernel(float *__restrict__ ga, float *__restrict__ gb, const float *__restrict__ g,
                               const float *__restrict__ a, const float *__restrict__ b, const StridedDesc d, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        int64_t rem = i, ao = 0, bo = 0;
        for (int k = d.ndim - 1; k >= 0; --k) {
            const int64_t c = rem % d.shape[k];
            rem /= d.shape[k];
            ao += c * d.a_strides[k];
            bo += c * d.b_strides[k];
        }
        const float gv = g[i], bv = b[bo];
        ga[i] = gv / bv;
        gb[i] = -gv * a[ao] / (bv * bv);
    }
}
int k_div_backward(float *ga, float *gb, const float *g, const float *a, const float *b, const StridedDesc &d) {
    MNI_TRY(ensure_init());
    int64_t n = 1;
    for (int i = 0; i < d.ndim; ++i) n *= d.shape[i];
    if (n <= 0) return MNI_OK;
    MNI_KERNEL_LAUNCH(div_bwd_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, ga, gb, g, a, b, d, n);
    return check_launch("div_backward");
}

// out[r, c] = a[r, c] + bias[c]   (src/native/kernels/elementwise.cu:43-47)
__global__ void add_bias_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ bias,
                                int64_t n, int64_t cols) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) out[i] = a[i] + bias[i % cols];
}
__global__ void add_bias4_kernel(float4 *__restrict__ out, const float4 *__restrict__ a,
                                 const float4 *__restrict__ bias, int64_t n4, int64_t cols4) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n4; i += step) {
        const float4 x = a[i], y = bias[i % cols4];
        out[i] = make_float4(x.x + y.x, x.y + y.y, x.z + y.z, x.w + y.w);
    }
}
int k_add_bias(float *out, const float *a, const float *bias, int64_t rows, int64_t cols) {
    const int64_t n = rows * cols;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (al16(out) && al16(a) && al16(bias) && (cols % 4) == 0) {
        MNI_KERNEL_LAUNCH(add_bias4_kernel, dim3(grid_for(n / 4, TPB * 2)), dim3(TPB), 0, ctx().stream,
                           reinterpret_cast<float4 *>(out), reinterpret_cast<const float4 *>(a),
                           reinterpret_cast<const float4 *>(bias), n / 4, cols / 4);
    } else {
        MNI_KERNEL_LAUNCH(add_bias_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, a, bias, n, cols);
    }
    return check_launch("add_bias");
}

// ---- unary ----------------------------------------------------------------------
__device__ __forceinline__ float un_apply(float x, int op, float s) {
    switch (op) {
    case UN_RELU: return fmaxf(x, 0.0f);  // f32::max(x, 0.0), activation.rs:116
    case UN_GELU: return d_gelu(x);
    case UN_NEG: return -x;
    case UN_SCALE: return x * s;
    case UN_EXP: return expf(x);                        // elementwise.rs:760-770
    case UN_LOG: return logf(x);                        // :839-849
    case UN_SIGMOID: return 1.0f / (1.0f + expf(-x));   // activation.rs:194-204
    case UN_POW: return powf(x, s);                     // elementwise.rs:1341-1351
    default: return x;
    }
}
__global__ void unary_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t n, int op, float s) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) out[i] = un_apply(x[i], op, s);
}
__global__ void unary4_kernel(float4 *__restrict__ out, const float4 *__restrict__ x, int64_t n4, int op, float s) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n4; i += step) {
        const float4 v = x[i];
        out[i] = make_float4(un_apply(v.x, op, s), un_apply(v.y, op, s), un_apply(v.z, op, s), un_apply(v.w, op, s));
    }
}
int k_unary(float *out, const float *x, int64_t n, int op, float s) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (al16(out) && al16(x) && (n % 4) == 0) {
        MNI_KERNEL_LAUNCH(unary4_kernel, dim3(grid_for(n / 4, TPB * 2)), dim3(TPB), 0, ctx().stream,
                           reinterpret_cast<float4 *>(out), reinterpret_cast<const float4 *>(x), n / 4, op, s);
    } else {
        MNI_KERNEL_LAUNCH(unary_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, x, n, op, s);
    }
    return check_launch("unary");
}

// relu_backward / gelu_backward (src/native/src/ops/activation.rs:74-84,154-164)
__global__ void unary_bwd_kernel(float *__restrict__ out, const float *__restrict__ g, const float *__restrict__ x,
                                 int64_t n, int op) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        const float xv = x[i], gv = g[i];
        out[i] = op == UN_RELU ? (xv > 0.0f ? gv : 0.0f) : gv * d_gelu_grad(xv);
    }
}
int k_unary_backward(float *out, const float *g, const float *x, int64_t n, int op) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(unary_bwd_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, g, x, n, op);
    return check_launch("unary_backward");
}

// exp / log / sigmoid / pow backward (elementwise.rs:800-809, 879-888, 1375-1386; activation.rs:231-241)
__global__ void unary2_bwd_kernel(float *__restrict__ out, const float *__restrict__ g, const float *__restrict__ saved,
                                  int64_t n, int op, float s) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        const float gv = g[i], v = saved[i];
        out[i] = op == UN_EXP ? gv * v : op == UN_LOG ? gv / v : op == UN_SIGMOID ? gv * v * (1.0f - v)
                                                               : gv * s * powf(v, s - 1.0f);
    }
}
int k_unary2_backward(float *out, const float *g, const float *saved, int64_t n, int op, float s) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(unary2_bwd_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, g, saved, n, op, s);
    return check_launch("unary2_backward");
}

// mul_backward for equal shapes (src/native/src/ops/elementwise.rs:348-390)
__global__ void mul_bwd_kernel(float *__restrict__ ga, float *__restrict__ gb, const float *__restrict__ g,
                               const float *__restrict__ a, const float *__restrict__ b, int64_t n) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        const float gv = g[i], av = a[i], bv = b[i];
        ga[i] = gv * bv;
        gb[i] = gv * av;
    }
}
int k_mul_backward_same(float *ga, float *gb, const float *g, const float *a, const float *b, int64_t n) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(mul_bwd_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, ga, gb, g, a, b, n);
    return check_launch("mul_backward");
}

// ---- column sum -------------------------------------------------------------------
// out[c] = sum_r a[r, c]: the bias gradient (unbroadcast of [rows, C] to [C],
// src/native/src/utils.rs:39-66) and the batch reduction of a broadcast matmul
// operand.  Two deterministic passes: row blocks into partials, then partials
// in block order.
static constexpr int CS_ROWS = 32;  // rows per block in pass 1 (a [4096, 768] gradient then gives 384 workgroups, not 96)
__global__ void colsum_partial_kernel(float *__restrict__ part, const float *__restrict__ a, int64_t rows,
                                      int64_t cols, int64_t rows_per_block) {
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= cols) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = min(rows, r0 + rows_per_block);
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int64_t r = r0;
    for (; r + 7 < r1; r += 8) {  // 8 loads in flight, four running sums
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = a[(r + e) * cols + c];
        s0 += v[0]; s1 += v[1]; s2 += v[2]; s3 += v[3];
        s0 += v[4]; s1 += v[5]; s2 += v[6]; s3 += v[7];
    }
    for (; r + 3 < r1; r += 4) {
        s0 += a[r * cols + c];
        s1 += a[(r + 1) * cols + c];
        s2 += a[(r + 2) * cols + c];
        s3 += a[(r + 3) * cols + c];
    }
    for (; r < r1; ++r) s0 += a[r * cols + c];
    part[(int64_t)blockIdx.y * cols + c] = (s0 + s1) + (s2 + s3);
}
// Few columns (a reduction to a scalar or to a short vector): a thread per
// column would leave most of a wavefront idle, so the 256 threads of a block
// form `lanes` = 256 / cols row lanes of cols threads each; row lane l takes
// rows l, l + lanes, ... of the block's CN_ROWS * lanes rows (consecutive
// threads read consecutive floats), and the lanes are added in lane order.
static constexpr int CN_COLS = 64;   // widest matrix that takes this form
static constexpr int CN_ROWS = 32;   // rows per thread
__global__ __launch_bounds__(256) void colsum_narrow_kernel(float *__restrict__ part, const float *__restrict__ a,
                                                            int64_t rows, int cols, int lanes) {
    __shared__ float sh[256];
    const int t = threadIdx.x;
    const int l = t / cols, c = t - l * cols;
    const int64_t r0 = (int64_t)blockIdx.x * CN_ROWS * lanes;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (l < lanes) {
#pragma unroll
        for (int i0 = 0; i0 < CN_ROWS; i0 += 8) {
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int64_t r = r0 + l + (int64_t)(i0 + e) * lanes;
                v[e] = r < rows ? a[r * cols + c] : 0.0f;
            }
            s0 += v[0]; s1 += v[1]; s2 += v[2]; s3 += v[3];
            s0 += v[4]; s1 += v[5]; s2 += v[6]; s3 += v[7];
        }
    }
    sh[t] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (t < cols) {
        float v = sh[t];
        for (int k = 1; k < lanes; ++k) v += sh[k * cols + t];
        part[(int64_t)blockIdx.x * cols + t] = v;
    }
}
// Pass 2: 64 columns per block, the partials dealt to four thread groups as
// contiguous quarters (a quarter of the loads per thread, all in flight at
// once for the usual few dozen partials); the four group sums are added in
// group order, so the result depends on the shape only.
static constexpr int CF_COLS = 64, CF_GROUPS = 4;
__global__ void colsum_final_kernel(float *__restrict__ out, const float *__restrict__ part, int64_t nparts,
                                    int64_t cols) {
    __shared__ float sums[CF_GROUPS][CF_COLS];
    const int cx = threadIdx.x % CF_COLS, grp = threadIdx.x / CF_COLS;
    const int64_t c = (int64_t)blockIdx.x * CF_COLS + cx;
    const int64_t per = (nparts + CF_GROUPS - 1) / CF_GROUPS;
    const int64_t p0 = min(nparts, grp * per), p1 = min(nparts, p0 + per);
    float s = 0.f;
    if (c < cols) {
        int64_t p = p0;
        for (; p + 7 < p1; p += 8) {  // 8 loads in flight, added in order
            float v[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = part[(p + e) * cols + c];
#pragma unroll
            for (int e = 0; e < 8; ++e) s += v[e];
        }
        for (; p < p1; ++p) s += part[p * cols + c];
    }
    sums[grp][cx] = s;
    __syncthreads();
    if (grp == 0 && c < cols) out[c] = ((sums[0][cx] + sums[1][cx]) + sums[2][cx]) + sums[3][cx];
}
static inline dim3 colsum_final_grid(int64_t cols) { return dim3((unsigned)((cols + CF_COLS - 1) / CF_COLS)); }
int k_colsum(float *out, const float *a, int64_t rows, int64_t cols) {
    if (cols <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (rows <= 0) return k_fill(out, 0.0f, cols);
    const dim3 block(TPB);
    // Row blocks: 32 rows each; more when the second grid axis (65535 blocks)
    // would not hold them.  Few columns and many rows: the row-lane form.
    const bool narrow = cols <= CN_COLS && rows >= 4 * CN_ROWS;
    // A few dozen rows (the strip sums a product's epilogue leaves for a bias gradient) are what the second pass
    // is made for: one launch, not a pass of 32-row blocks and then their sum.
    if (!narrow && rows > CS_ROWS && rows <= 256) {
        MNI_KERNEL_LAUNCH(colsum_final_kernel, colsum_final_grid(cols), dim3(CF_COLS * CF_GROUPS), 0, ctx().stream, out, a, rows, cols);
        return check_launch("colsum_final");
    }
    const int lanes = narrow ? 256 / (int)cols : 0;
    int64_t rows_per_block = narrow ? (int64_t)CN_ROWS * lanes : CS_ROWS;
    int64_t nparts = (rows + rows_per_block - 1) / rows_per_block;
    if (!narrow && nparts > 65535) {
        rows_per_block = ((rows + 65534) / 65535 + 7) / 8 * 8;
        nparts = (rows + rows_per_block - 1) / rows_per_block;
    }
    if (nparts > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "colsum: too many rows (%lld)", (long long)rows);
    const unsigned gx = (unsigned)((cols + TPB - 1) / TPB);
    void *part = nullptr;
    if (nparts > 1) MNI_TRY(dev_alloc(&part, (size_t)nparts * cols * sizeof(float)));
    float *dst = nparts > 1 ? (float *)part : out;
    if (narrow)
        MNI_KERNEL_LAUNCH(colsum_narrow_kernel, dim3((unsigned)nparts), dim3(256), 0, ctx().stream, dst, a, rows, (int)cols, lanes);
    else
        MNI_KERNEL_LAUNCH(colsum_partial_kernel, dim3(gx, (unsigned)nparts), block, 0, ctx().stream, dst, a, rows, cols, rows_per_block);
    int rc = check_launch("colsum_partial");
    if (rc == MNI_OK && nparts > 1) {
        if (nparts > 1024) {
            // many partials: they are a tall matrix themselves
            rc = k_colsum(out, (const float *)part, nparts, cols);
        } else {
            MNI_KERNEL_LAUNCH(colsum_final_kernel, colsum_final_grid(cols), dim3(CF_COLS * CF_GROUPS), 0, ctx().stream, out, (const float *)part, nparts, cols);
            rc = check_launch("colsum_final");
        }
    }
    if (part) dev_free(part);
    return rc;
}

// ---- fused bias + GELU (src/native/src/ops/fused.rs:247-273, 316-351) ------------------
// forward: out = gelu(x + bias[col]); backward: dx = g * gelu'(x + bias[col])
// and dbias = column sums of dx, taken in the same pass over row blocks
// (partials per block, summed in block order: deterministic).
__global__ void bias_gelu_kernel(float *__restrict__ out, const float *__restrict__ x, const float *__restrict__ bias,
                                 int64_t n, int64_t cols) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) out[i] = d_gelu(x[i] + bias[i % cols]);
}
__global__ void bias_gelu4_kernel(float4 *__restrict__ out, const float4 *__restrict__ x, const float4 *__restrict__ bias,
                                  int64_t n4, int64_t cols4) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n4; i += step) {
        const float4 v = x[i], b = bias[i % cols4];
        out[i] = make_float4(d_gelu(v.x + b.x), d_gelu(v.y + b.y), d_gelu(v.z + b.z), d_gelu(v.w + b.w));
    }
}
int k_bias_gelu(float *out, const float *x, const float *bias, int64_t rows, int64_t cols) {
    const int64_t n = rows * cols;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (cols % 4 == 0 && al16(out) && al16(x) && al16(bias))
        MNI_KERNEL_LAUNCH(bias_gelu4_kernel, dim3(grid_for(n / 4, TPB * 2)), dim3(TPB), 0, ctx().stream, (float4 *)out,
                           (const float4 *)x, (const float4 *)bias, n / 4, cols / 4);
    else
        MNI_KERNEL_LAUNCH(bias_gelu_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, x, bias, n, cols);
    return check_launch("bias_gelu");
}
static constexpr int BG_ROWS = 16;  // rows per block in the backward pass
template <typename V, int W>
__global__ void bias_gelu_bwd_kernel(V *__restrict__ dx, V *__restrict__ part, const V *__restrict__ g,
                                     const V *__restrict__ x, const V *__restrict__ bias, int64_t rows, int64_t colsv,
                                     int64_t rows_per_block) {
    // colsv = columns in units of V (float or float4); thread = one V column, rows_per_block rows
    const int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (c >= colsv) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = min(rows, r0 + rows_per_block);
    float b[W], s[W];
    {
        const V bv = bias[c];
        const float *bp = reinterpret_cast<const float *>(&bv);
#pragma unroll
        for (int e = 0; e < W; ++e) { b[e] = bp[e]; s[e] = 0.f; }
    }
    for (int64_t r = r0; r < r1; ++r) {
        const V gv = g[r * colsv + c], xv = x[r * colsv + c];
        const float *gp = reinterpret_cast<const float *>(&gv), *xp = reinterpret_cast<const float *>(&xv);
        V ov;
        float *op = reinterpret_cast<float *>(&ov);
#pragma unroll
        for (int e = 0; e < W; ++e) {
            op[e] = gp[e] * d_gelu_grad(xp[e] + b[e]);
            s[e] += op[e];
        }
        dx[r * colsv + c] = ov;
    }
    V sv;
    float *sp = reinterpret_cast<float *>(&sv);
#pragma unroll
    for (int e = 0; e < W; ++e) sp[e] = s[e];
    part[(int64_t)blockIdx.y * colsv + c] = sv;
}
int k_bias_gelu_backward(float *dx, float *dbias, const float *g, const float *x, const float *bias, int64_t rows,
                         int64_t cols) {
    if (cols <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (rows <= 0) return k_fill(dbias, 0.0f, cols);
    int64_t rows_per_block = BG_ROWS;
    int64_t nparts = (rows + rows_per_block - 1) / rows_per_block;
    if (nparts > 65535) {  // the second grid axis holds no more
        rows_per_block = (rows + 65534) / 65535;
        nparts = (rows + rows_per_block - 1) / rows_per_block;
    }
    const bool vec = cols % 4 == 0 && al16(dx) && al16(g) && al16(x) && al16(bias) && al16(dbias);
    const int64_t colsv = vec ? cols / 4 : cols;
    const dim3 block(TPB);
    const unsigned gx = (unsigned)((colsv + TPB - 1) / TPB);
    void *part = nullptr;
    if (nparts > 1) MNI_TRY(dev_alloc(&part, (size_t)nparts * cols * sizeof(float)));
    float *dst = nparts > 1 ? (float *)part : dbias;
    if (vec)
        MNI_KERNEL_LAUNCH((bias_gelu_bwd_kernel<float4, 4>), dim3(gx, (unsigned)nparts), block, 0, ctx().stream, (float4 *)dx,
                           (float4 *)dst, (const float4 *)g, (const float4 *)x, (const float4 *)bias, rows, colsv, rows_per_block);
    else
        MNI_KERNEL_LAUNCH((bias_gelu_bwd_kernel<float, 1>), dim3(gx, (unsigned)nparts), block, 0, ctx().stream, dx, dst, g, x,
                           bias, rows, colsv, rows_per_block);
    int rc = check_launch("bias_gelu_backward");
    if (rc == MNI_OK && nparts > 1) {
        MNI_KERNEL_LAUNCH(colsum_final_kernel, colsum_final_grid(cols), dim3(CF_COLS * CF_GROUPS), 0, ctx().stream, dbias,
                           (const float *)part, nparts, cols);
        rc = check_launch("colsum_final");
    }
    if (part) dev_free(part);
    return rc;
}

// ---- max along one dim (src/native/src/ops/reduce.rs:333-368, 416-447) --------------------
__global__ void max_dim_kernel(float *__restrict__ out, const float *__restrict__ a, int64_t outer, int64_t dim,
                               int64_t inner) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t o = idx / inner, i = idx - o * inner;
    const float *p = a + o * dim * inner + i;
    float m = -INFINITY;
    for (int64_t d = 0; d < dim; ++d) {
        const float v = p[d * inner];
        if (v > m) m = v;  // strict >, like the reference (a NaN never replaces the maximum)
    }
    out[idx] = m;
}
__global__ void max_rows_kernel(float *__restrict__ out, const float *__restrict__ a, int64_t outer, int64_t dim) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= outer) return;
    const float *p = a + row * dim;
    float m = -INFINITY;
    for (int64_t d = lane; d < dim; d += 64) {
        const float v = p[d];
        if (v > m) m = v;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o = __shfl_xor(m, off, 64);
        if (o > m) m = o;
    }
    if (lane == 0) out[row] = m;
}
// A long reduced axis under few outputs, in two levels (a maximum does not depend on the order it is taken in): the
// axis is cut into `parts` blocks of `blk`, a thread takes the maximum of one block for one output, and the block
// maxima are a shorter axis for the forms above.  (One thread per output walked a million rows alone: 90 ms.)
__global__ void max_dim_blocks_kernel(float *__restrict__ part, const float *__restrict__ a, int64_t outer, int64_t dim, int64_t inner,
                                      int64_t blk, int64_t parts) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * parts * inner) return;
    const int64_t i = idx % inner, op = idx / inner, p = op % parts, o = op / parts;
    const int64_t d0 = p * blk, d1 = min(dim, d0 + blk);
    const float *q = a + o * dim * inner + i;
    float m = -INFINITY;
    for (int64_t d = d0; d < d1; ++d) {
        const float v = q[d * inner];
        if (v > m) m = v;
    }
    part[idx] = m;
}
// The same for a few long contiguous rows: a wavefront per chunk of a row, lanes striding it.
static constexpr int64_t MC_CHUNK = 8192;
__global__ void max_chunks_kernel(float *__restrict__ part, const float *__restrict__ a, int64_t total, int64_t dim, int64_t chunks,
                                  int64_t chunk) {
    const int lane = threadIdx.x & 63;
    const int64_t idx = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (idx >= total) return;
    const int64_t o = idx / chunks, c = idx - o * chunks;
    const int64_t len = min(chunk, dim - c * chunk);
    const float *p = a + o * dim + c * chunk;
    float m = -INFINITY;
    for (int64_t d = lane; d < len; d += 64) {
        const float v = p[d];
        if (v > m) m = v;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float o2 = __shfl_xor(m, off, 64);
        if (o2 > m) m = o2;
    }
    if (lane == 0) part[idx] = m;
}
int k_max_dim(float *out, const float *a, int64_t outer, int64_t dim, int64_t inner) {
    const int64_t n = outer * inner;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (inner == 1 && outer < 4096 && (dim >= 4 * MC_CHUNK || (dim >= MC_CHUNK && outer <= 512))) {
        const int64_t chunk = dim >= 4 * MC_CHUNK ? MC_CHUNK : MC_CHUNK / 8;
        const int64_t chunks = (dim + chunk - 1) / chunk, total = outer * chunks;
        void *part = nullptr;
        MNI_TRY(dev_alloc(&part, (size_t)total * sizeof(float)));
        MNI_KERNEL_LAUNCH(max_chunks_kernel, dim3(grid_for(total, 4)), dim3(TPB), 0, ctx().stream, (float *)part, a, total, dim, chunks, chunk);
        int rc = check_launch("max_chunks");
        if (rc == MNI_OK) rc = k_max_dim(out, (const float *)part, outer, chunks, 1);
        dev_free(part);
        return rc;
    }
    if (inner > 1 && n < 32768 && dim >= 2048) {
        const int64_t want = (1 << 17) / n;                      // blocks per output for ~128 K threads
        const int64_t blk = max((int64_t)32, (dim + want - 1) / want), parts = (dim + blk - 1) / blk;
        if (parts > 1) {
            void *part = nullptr;
            MNI_TRY(dev_alloc(&part, (size_t)(outer * parts * inner) * sizeof(float)));
            MNI_KERNEL_LAUNCH(max_dim_blocks_kernel, dim3(grid_for(outer * parts * inner, TPB)), dim3(TPB), 0, ctx().stream, (float *)part, a,
                               outer, dim, inner, blk, parts);
            int rc = check_launch("max_dim_blocks");
            if (rc == MNI_OK) rc = k_max_dim(out, (const float *)part, outer, parts, inner);
            dev_free(part);
            return rc;
        }
    }
    if (inner == 1 && dim >= 256)
        MNI_KERNEL_LAUNCH(max_rows_kernel, dim3(grid_for(outer, 4)), dim3(TPB), 0, ctx().stream, out, a, outer, dim);
    else
        MNI_KERNEL_LAUNCH(max_dim_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx().stream, out, a, outer, dim, inner);
    return check_launch("max_dim");
}
__global__ void max_bwd_kernel(float *__restrict__ out, const float *__restrict__ x, const float *__restrict__ mx,
                               const float *__restrict__ g, int64_t dim, int64_t inner, int64_t n) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n; idx += step) {
        const int64_t o = idx / (dim * inner), i = idx % inner;
        const int64_t mi = o * inner + i;
        out[idx] = fabsf(x[idx] - mx[mi]) < 1e-6f ? g[mi] : 0.0f;
    }
}
int k_max_backward(float *out, const float *x, const float *mx, const float *g, int64_t outer, int64_t dim, int64_t inner) {
    const int64_t n = outer * dim * inner;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(max_bwd_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, x, mx, g, dim, inner, n);
    return check_launch("max_backward");
}

// ---- layernorm over the last extent (src/native/src/ops/norm.rs:167-215, 273-322) -------------
// One wavefront per row: mean, biased variance (second pass over the centred
// values, as the reference), rstd = 1 / sqrt(var / c + eps).
__device__ __forceinline__ float ew_wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__global__ void layernorm_kernel(float *__restrict__ out, float *__restrict__ mean, float *__restrict__ rstd,
                                 const float *__restrict__ x, const float *__restrict__ gamma,
                                 const float *__restrict__ beta, int64_t rows, int64_t c, float eps) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *p = x + row * c;
    float s = 0.f;
    for (int64_t j = lane; j < c; j += 64) s += p[j];
    const float m = ew_wave_sum(s) / (float)c;
    float v = 0.f;
    for (int64_t j = lane; j < c; j += 64) { const float d = p[j] - m; v += d * d; }
    const float r = 1.0f / sqrtf(ew_wave_sum(v) / (float)c + eps);
    for (int64_t j = lane; j < c; j += 64) out[row * c + j] = (p[j] - m) * r * gamma[j] + beta[j];
    if (lane == 0) { mean[row] = m; rstd[row] = r; }
}
// Rows of 1024 to 16384 values in whole 16-byte pieces: a workgroup per row holds the row in registers -- one
// read, one write, two LDS reductions (a wavefront walked a 4096-wide row 64 steps at a time, three times over:
// 21 us for a single row).  RESIDUAL: the row is x + residual, which is also written out (res).
template <int NV, bool RESIDUAL>
__global__ __launch_bounds__(256) void layernorm_wg_kernel(float *__restrict__ out, float *__restrict__ res, float *__restrict__ mean,
                                                           float *__restrict__ rstd, const float *__restrict__ x,
                                                           const float *__restrict__ residual, const float *__restrict__ gamma,
                                                           const float *__restrict__ beta, int64_t c, float eps) {
    __shared__ float red[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row = blockIdx.x, c4 = c >> 2;
    const float4 *p = reinterpret_cast<const float4 *>(x + row * c);
    float4 v[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t j = tid + 256 * i;
        v[i] = j < c4 ? p[j] : make_float4(0.f, 0.f, 0.f, 0.f);
    }
    if (RESIDUAL) {
        const float4 *q = reinterpret_cast<const float4 *>(residual + row * c);
        float4 *ps = reinterpret_cast<float4 *>(res + row * c);
#pragma unroll
        for (int i = 0; i < NV; ++i) {
            const int64_t j = tid + 256 * i;
            if (j < c4) {
                const float4 r4 = q[j];
                v[i].x += r4.x; v[i].y += r4.y; v[i].z += r4.z; v[i].w += r4.w;
                ps[j] = v[i];
            }
        }
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) { s += v[i].x; s += v[i].y; s += v[i].z; s += v[i].w; }  // (pieces past the row are zeros)
    s = ew_wave_sum(s);
    if (lane == 0) red[0][wave] = s;
    __syncthreads();
    const float m = ((red[0][0] + red[0][1]) + (red[0][2] + red[0][3])) / (float)c;
    float var = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        if (tid + 256 * i < c4) {
            const float dx = v[i].x - m, dy = v[i].y - m, dz = v[i].z - m, dw = v[i].w - m;
            var += dx * dx; var += dy * dy; var += dz * dz; var += dw * dw;
        }
    }
    var = ew_wave_sum(var);
    if (lane == 0) red[1][wave] = var;
    __syncthreads();
    const float r = 1.0f / sqrtf(((red[1][0] + red[1][1]) + (red[1][2] + red[1][3])) / (float)c + eps);
    const float4 *g4 = reinterpret_cast<const float4 *>(gamma), *b4 = reinterpret_cast<const float4 *>(beta);
    float4 *o = reinterpret_cast<float4 *>(out + row * c);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t j = tid + 256 * i;
        if (j < c4) {
            const float4 gg = g4[j], bb = b4[j];
            o[j] = make_float4((v[i].x - m) * r * gg.x + bb.x, (v[i].y - m) * r * gg.y + bb.y, (v[i].z - m) * r * gg.z + bb.z,
                               (v[i].w - m) * r * gg.w + bb.w);
        }
    }
    if (tid == 0) { mean[row] = m; rstd[row] = r; }
}
// Launches the form above when the row fits it; false when it does not.
bool launch_layernorm_workgroups(float *out, float *res, float *mean, float *rstd, const float *x, const float *residual,
                                 const float *gamma, const float *beta, int64_t rows, int64_t c, float eps) {
    if (c < 1024 || c > 16384 || c % 4 != 0 || rows > 0x7fffffffLL) return false;
    if (!al16(out) || !al16(x) || !al16(gamma) || !al16(beta) || (residual && (!al16(residual) || !al16(res)))) return false;
    const dim3 grid((unsigned)rows), block(256);
    hipStream_t st = ctx().stream;
    if (residual && c <= 2048) MNI_KERNEL_LAUNCH((layernorm_wg_kernel<2, true>), grid, block, 0, st, out, res, mean, rstd, x, residual, gamma, beta, c, eps);
    else if (residual && c <= 8192) MNI_KERNEL_LAUNCH((layernorm_wg_kernel<8, true>), grid, block, 0, st, out, res, mean, rstd, x, residual, gamma, beta, c, eps);
    else if (residual) MNI_KERNEL_LAUNCH((layernorm_wg_kernel<16, true>), grid, block, 0, st, out, res, mean, rstd, x, residual, gamma, beta, c, eps);
    else if (c <= 2048) MNI_KERNEL_LAUNCH((layernorm_wg_kernel<2, false>), grid, block, 0, st, out, res, mean, rstd, x, residual, gamma, beta, c, eps);
    else if (c <= 8192) MNI_KERNEL_LAUNCH((layernorm_wg_kernel<8, false>), grid, block, 0, st, out, res, mean, rstd, x, residual, gamma, beta, c, eps);
    else MNI_KERNEL_LAUNCH((layernorm_wg_kernel<16, false>), grid, block, 0, st, out, res, mean, rstd, x, residual, gamma, beta, c, eps);
    return true;
}
int k_layernorm(float *out, float *mean, float *rstd, const float *x, const float *gamma, const float *beta, int64_t rows,
                int64_t c, float eps) {
    if (rows <= 0 || c <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (launch_layernorm_workgroups(out, nullptr, mean, rstd, x, nullptr, gamma, beta, rows, c, eps)) return check_launch("layernorm");
    MNI_KERNEL_LAUNCH(layernorm_kernel, dim3(grid_for(rows, 4)), dim3(TPB), 0, ctx().stream, out, mean, rstd, x, gamma, beta,
                       rows, c, eps);
    return check_launch("layernorm");
}
// dx per row (one wavefront per row)
__global__ void layernorm_bwd_rows_kernel(float *__restrict__ dx, const float *__restrict__ g, const float *__restrict__ x,
                                          const float *__restrict__ gamma, const float *__restrict__ mean,
                                          const float *__restrict__ rstd, int64_t rows, int64_t c) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float m = mean[row], r = rstd[row];
    const float *px = x + row * c, *pg = g + row * c;
    float sum_dg = 0.f, sum_dgx = 0.f;
    for (int64_t j = lane; j < c; j += 64) {
        const float xhat = (px[j] - m) * r, dg = pg[j] * gamma[j];
        sum_dg += dg;
        sum_dgx += dg * xhat;
    }
    sum_dg = ew_wave_sum(sum_dg);
    sum_dgx = ew_wave_sum(sum_dgx);
    for (int64_t j = lane; j < c; j += 64) {
        const float xhat = (px[j] - m) * r, dg = pg[j] * gamma[j];
        dx[row * c + j] = r * (dg - sum_dg / (float)c - xhat * sum_dgx / (float)c);
    }
}
// dgamma / dbeta: column sums of g * xhat and g over row blocks, partials summed in block order
__global__ void layernorm_bwd_cols_kernel(float *__restrict__ pgamma, float *__restrict__ pbeta, const float *__restrict__ g,
                                          const float *__restrict__ x, const float *__restrict__ mean,
                                          const float *__restrict__ rstd, int64_t rows, int64_t c, int64_t rows_per_block) {
    const int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (j >= c) return;
    const int64_t r0 = (int64_t)blockIdx.y * rows_per_block;
    const int64_t r1 = min(rows, r0 + rows_per_block);
    float sg = 0.f, sb = 0.f;
    for (int64_t r = r0; r < r1; ++r) {
        const float gv = g[r * c + j];
        sg += gv * ((x[r * c + j] - mean[r]) * rstd[r]);
        sb += gv;
    }
    pgamma[(int64_t)blockIdx.y * c + j] = sg;
    pbeta[(int64_t)blockIdx.y * c + j] = sb;
}
int k_layernorm_backward(float *dx, float *dgamma, float *dbeta, const float *g, const float *x, const float *gamma,
                         const float *mean, const float *rstd, int64_t rows, int64_t c) {
    if (c <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (rows <= 0) { MNI_TRY(k_fill(dgamma, 0.0f, c)); return k_fill(dbeta, 0.0f, c); }
    MNI_KERNEL_LAUNCH(layernorm_bwd_rows_kernel, dim3(grid_for(rows, 4)), dim3(TPB), 0, ctx().stream, dx, g, x, gamma, mean,
                       rstd, rows, c);
    MNI_TRY(check_launch("layernorm_backward_rows"));
    // row blocks of BG_ROWS; more rows per block when the second grid axis (65535 blocks) would not hold them all
    int64_t rows_per_block = BG_ROWS;
    if ((rows + rows_per_block - 1) / rows_per_block > 65535) rows_per_block = (rows + 65534) / 65535;
    const int64_t nparts = (rows + rows_per_block - 1) / rows_per_block;
    void *part = nullptr;
    MNI_TRY(dev_alloc(&part, (size_t)2 * nparts * c * sizeof(float)));
    float *pg = (float *)part, *pb = pg + nparts * c;
    const unsigned gx = (unsigned)((c + TPB - 1) / TPB);
    MNI_KERNEL_LAUNCH(layernorm_bwd_cols_kernel, dim3(gx, (unsigned)nparts), dim3(TPB), 0, ctx().stream, pg, pb, g, x, mean,
                       rstd, rows, c, rows_per_block);
    int rc = check_launch("layernorm_backward_cols");
    if (rc == MNI_OK) {
        MNI_KERNEL_LAUNCH(colsum_final_kernel, colsum_final_grid(c), dim3(CF_COLS * CF_GROUPS), 0, ctx().stream, dgamma, (const float *)pg, nparts, c);
        MNI_KERNEL_LAUNCH(colsum_final_kernel, colsum_final_grid(c), dim3(CF_COLS * CF_GROUPS), 0, ctx().stream, dbeta, (const float *)pb, nparts, c);
        rc = check_launch("colsum_final");
    }
    dev_free(part);
    return rc;
}

// ---- reduce / expand along one dim ----------------------------------------------------
// sum / mean along `dim` (src/native/src/ops/reduce.rs:13-46,169-184): input
// viewed as [outer, dim, inner].
__global__ void reduce_inner_kernel(float *__restrict__ out, const float *__restrict__ a, int64_t outer, int64_t dim,
                                    int64_t inner, float div) {
    // one thread per output, consecutive threads along `inner` (coalesced);
    // terms are added in increasing d like the reference's flat-order loop.
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t o = idx / inner, i = idx - o * inner;
    const float *p = a + o * dim * inner + i;
    float s = 0.f;
    for (int64_t d = 0; d < dim; ++d) s += p[d * inner];
    out[idx] = s / div;
}
__global__ void reduce_rows_kernel(float *__restrict__ out, const float *__restrict__ a, int64_t outer, int64_t dim,
                                   float div) {
    // inner == 1: one wavefront per row, lanes stride the row.
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= outer) return;
    const float *p = a + row * dim;
    float s = 0.f;
    for (int64_t d = lane; d < dim; d += 64) s += p[d];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == 0) out[row] = s / div;
}
// A few long rows (the sum of a whole tensor: one row of millions): a wavefront per chunk of a row first, the
// chunk sums are a short matrix for the forms above.  Lanes stride the chunk, 8 loads in flight, four running
// sums folded in a fixed order.
static constexpr int64_t RC_CHUNK = 8192;
__global__ void reduce_chunks_kernel(float *__restrict__ part, const float *__restrict__ a, int64_t nchunks_total, int64_t dim,
                                     int64_t chunks, int64_t chunk) {
    const int lane = threadIdx.x & 63;
    const int64_t idx = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (idx >= nchunks_total) return;
    const int64_t o = idx / chunks, c = idx - o * chunks;
    const int64_t len = min(chunk, dim - c * chunk);
    const float *p = a + o * dim + c * chunk;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    int64_t d = lane;
    for (; d + 7 * 64 < len; d += 8 * 64) {
        float v[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = p[d + e * 64];
        s0 += v[0]; s1 += v[1]; s2 += v[2]; s3 += v[3];
        s0 += v[4]; s1 += v[5]; s2 += v[6]; s3 += v[7];
    }
    for (; d < len; d += 64) s0 += p[d];
    float s = (s0 + s1) + (s2 + s3);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == 0) part[idx] = s;
}
__global__ void div_inplace_kernel(float *__restrict__ x, float div, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) x[i] = x[i] / div;
}
int k_reduce_dim(float *out, const float *a, int64_t outer, int64_t dim, int64_t inner, float div) {
    const int64_t n = outer * inner;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (inner == 1 && outer < 4096 && (dim >= 4 * RC_CHUNK || (dim >= RC_CHUNK && outer <= 512))) {
        // (a wavefront per row would leave the few rows to a few wavefronts: 16 M elements in one row took 58 ms,
        // 8 rows of 16384 27 us; shorter chunks for the shorter rows)
        const int64_t chunk = dim >= 4 * RC_CHUNK ? RC_CHUNK : RC_CHUNK / 8;
        const int64_t chunks = (dim + chunk - 1) / chunk, total = outer * chunks;
        void *part = nullptr;
        MNI_TRY(dev_alloc(&part, (size_t)total * sizeof(float)));
        MNI_KERNEL_LAUNCH(reduce_chunks_kernel, dim3(grid_for(total, 4)), dim3(TPB), 0, ctx().stream, (float *)part, a, total, dim, chunks, chunk);
        int rc = check_launch("reduce_chunks");
        if (rc == MNI_OK) rc = k_reduce_dim(out, (const float *)part, outer, chunks, 1, div);
        dev_free(part);
        return rc;
    }
    if (inner > 1 && dim >= 256 && n < 32768 && outer <= 64) {
        // Few outputs under a long reduced axis (the column sums of a tall matrix): a thread per output would
        // walk the axis alone (4096 x 4096 summed over its rows: 977 us); the two-pass column sum per outer slice.
        for (int64_t o = 0; o < outer; ++o) MNI_TRY(k_colsum(out + o * inner, a + o * dim * inner, dim, inner));
        if (div != 1.0f) {
            MNI_KERNEL_LAUNCH(div_inplace_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx().stream, out, div, n);
            return check_launch("div_inplace");
        }
        return MNI_OK;
    }
    if (inner == 1 && dim >= 256) {
        MNI_KERNEL_LAUNCH(reduce_rows_kernel, dim3(grid_for(outer, 4)), dim3(TPB), 0, ctx().stream, out, a, outer, dim, div);
        return check_launch("reduce_rows");
    }
    MNI_KERNEL_LAUNCH(reduce_inner_kernel, dim3(grid_for(n, TPB)), dim3(TPB), 0, ctx().stream, out, a, outer, dim, inner, div);
    return check_launch("reduce_inner");
}

// ---- mean of squared differences along the last dim, one pass each way ------------------------------------
// What mseLoss composes from sub, mul and two means (src/nn.ts:161-165; the second mean runs over the size-1 dim
// the first one leaves, so the loss is one value per row): out[r] = sum_c (p[r, c] - t[r, c])^2 / dim.
// One wavefront per row, lanes stride the row (16-byte pieces when the row allows), sums folded in a fixed order.
// `seeded` (may be null): the gradient for an upstream gradient of all ones, written in the same pass with the
// arithmetic of the backward kernels below, so that a backward() rooted at this loss has nothing left to launch.
__global__ void mse_rows_kernel(float *__restrict__ out, const float *__restrict__ p, const float *__restrict__ t, int64_t rows,
                                int64_t dim, float div, int vec, float *__restrict__ seeded) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *pr = p + row * dim, *tr = t + row * dim;
    float *sr = seeded ? seeded + row * dim : nullptr;
    const float gr = 1.0f / div;
    float s = 0.f;
    if (vec) {
        const int64_t n4 = dim >> 2;
        for (int64_t d = lane; d < n4; d += 64) {
            const float4 a = reinterpret_cast<const float4 *>(pr)[d], b = reinterpret_cast<const float4 *>(tr)[d];
            const float x = a.x - b.x, y = a.y - b.y, z = a.z - b.z, w = a.w - b.w;
            s += x * x; s += y * y; s += z * z; s += w * w;
            if (sr) {
                float4 o;
                o.x = gr * x; o.y = gr * y; o.z = gr * z; o.w = gr * w;
                o.x *= 2.0f; o.y *= 2.0f; o.z *= 2.0f; o.w *= 2.0f;
                reinterpret_cast<float4 *>(sr)[d] = o;
            }
        }
    } else {
        for (int64_t d = lane; d < dim; d += 64) {
            const float x = pr[d] - tr[d];
            s += x * x;
            if (sr) sr[d] = 2.0f * (gr * x);
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == 0) out[row] = s / div;
}
int k_mse_rows(float *out, const float *p, const float *t, int64_t rows, int64_t dim, float *seeded) {
    if (rows <= 0) return MNI_OK;
    if (dim <= 0) return set_error(MNI_ERR_INVALID, "mse: empty rows");
    MNI_TRY(ensure_init());
    const int vec = dim % 4 == 0 && (((uintptr_t)p | (uintptr_t)t | (uintptr_t)seeded) & 15) == 0;
    MNI_KERNEL_LAUNCH(mse_rows_kernel, dim3(grid_for(rows, 4)), dim3(TPB), 0, ctx().stream, out, p, t, rows, dim, (float)dim, vec, seeded);
    return check_launch("mse_rows");
}
// Its backward in one pass: what mean_backward (g / dim), mul_backward (g d for each of the two operands, added up) and
// sub_backward (the negative for the target) leave behind: dp[r, c] = (g[r] / dim) d + (g[r] / dim) d with
// d = p - t, and dt = -dp when it is wanted.
__global__ void mse_rows_backward_kernel(float *__restrict__ dp, float *__restrict__ dt, const float *__restrict__ p,
                                         const float *__restrict__ t, const float *__restrict__ g, int64_t dim, float div, int64_t n) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n; idx += step) {
        const float gr = g[idx / dim] / div;
        const float v = gr * (p[idx] - t[idx]);
        const float o = 2.0f * v;  // (v + v, out of reach of a contraction into one fused multiply-add)
        dp[idx] = o;
        if (dt) dt[idx] = -o;
    }
}
__global__ void mse_rows_backward4_kernel(float4 *__restrict__ dp, float4 *__restrict__ dt, const float4 *__restrict__ p,
                                          const float4 *__restrict__ t, const float *__restrict__ g, int64_t dim4, float div, int64_t n4) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n4; idx += step) {
        const float gr = g[idx / dim4] / div;
        const float4 a = p[idx], b = t[idx];
        float4 o;
        o.x = gr * (a.x - b.x); o.y = gr * (a.y - b.y); o.z = gr * (a.z - b.z); o.w = gr * (a.w - b.w);
        o.x *= 2.0f; o.y *= 2.0f; o.z *= 2.0f; o.w *= 2.0f;  // (v + v, out of reach of a contraction into one fused multiply-add)
        dp[idx] = o;
        if (dt) dt[idx] = make_float4(-o.x, -o.y, -o.z, -o.w);
    }
}
int k_mse_rows_backward(float *dp, float *dt, const float *p, const float *t, const float *g, int64_t rows, int64_t dim) {
    const int64_t n = rows * dim;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    const bool al = (((uintptr_t)dp | (uintptr_t)dt | (uintptr_t)p | (uintptr_t)t) & 15) == 0;
    if (dim % 4 == 0 && al) {
        MNI_KERNEL_LAUNCH(mse_rows_backward4_kernel, dim3(grid_for(n / 4, TPB)), dim3(TPB), 0, ctx().stream, (float4 *)dp, (float4 *)dt,
                          (const float4 *)p, (const float4 *)t, g, dim / 4, (float)dim, n / 4);
        return check_launch("mse_rows_backward4");
    }
    MNI_KERNEL_LAUNCH(mse_rows_backward_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, dp, dt, p, t, g, dim, (float)dim, n);
    return check_launch("mse_rows_backward");
}

// sum_backward / mean_backward (src/native/src/ops/reduce.rs:94-118,232-263)
__global__ void expand_dim_kernel(float *__restrict__ out, const float *__restrict__ g, int64_t outer, int64_t dim,
                                  int64_t inner, float div, int64_t n) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n; idx += step) {
        const int64_t o = idx / (dim * inner);
        const int64_t i = idx % inner;
        out[idx] = g[o * inner + i] / div;
    }
}
int k_expand_dim(float *out, const float *g, int64_t outer, int64_t dim, int64_t inner, float div) {
    const int64_t n = outer * dim * inner;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(expand_dim_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, out, g, outer, dim, inner, div, n);
    return check_launch("expand_dim");
}

// ---- generic unbroadcast ----------------------------------------------------------------
// One thread per output element; it walks the broadcast coordinates in the
// reference's flat order (src/native/src/utils.rs:55-64), so the sum order per
// element is the reference's.
struct UnbDesc {
    int gnd;                          // grad dims
    int64_t gshape[MNI_MAX_DIMS];
    int64_t gstr[MNI_MAX_DIMS];
    int64_t oshape_al[MNI_MAX_DIMS];  // orig shape right-aligned to gnd (1 where missing)
    int nred;                         // reduced dims, outermost first
    int red_dim[MNI_MAX_DIMS];
};
__global__ void unbroadcast_kernel(float *__restrict__ out, const float *__restrict__ g, const UnbDesc d, int64_t on,
                                   int64_t red_total) {
    const int64_t oi = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (oi >= on) return;
    // base offset in g from the output coordinate
    int64_t rem = oi, base = 0;
    for (int k = d.gnd - 1; k >= 0; --k) {
        const int64_t ext = d.oshape_al[k];
        const int64_t c = rem % ext;
        rem /= ext;
        base += c * d.gstr[k];
    }
    float s = 0.f;
    for (int64_t t = 0; t < red_total; ++t) {
        int64_t r = t, off = 0;
        for (int k = d.nred - 1; k >= 0; --k) {
            const int dim = d.red_dim[k];
            const int64_t c = r % d.gshape[dim];
            r /= d.gshape[dim];
            off += c * d.gstr[dim];
        }
        s += g[base + off];
    }
    out[oi] = s;
}
int k_unbroadcast(float *out, const float *g, const int64_t *gshape, int gnd, const int64_t *oshape, int ond) {
    MNI_TRY(ensure_init());
    if (gnd > MNI_MAX_DIMS || ond > gnd) return set_error(MNI_ERR_INVALID, "unbroadcast: bad ranks %d -> %d", gnd, ond);
    UnbDesc d;
    d.gnd = gnd;
    int64_t gs = 1;
    for (int k = gnd - 1; k >= 0; --k) { d.gshape[k] = gshape[k]; d.gstr[k] = gs; gs *= gshape[k]; }
    const int off = gnd - ond;
    int64_t on = 1, red_total = 1;
    d.nred = 0;
    for (int k = 0; k < gnd; ++k) {
        const int64_t ext = k < off ? 1 : oshape[k - off];
        d.oshape_al[k] = ext;
        on *= ext;
        if (ext == 1 && gshape[k] != 1) { d.red_dim[d.nred++] = k; red_total *= gshape[k]; }
        else if (ext != gshape[k]) return set_error(MNI_ERR_INVALID, "unbroadcast: shapes do not broadcast");
    }
    if (on <= 0) return MNI_OK;
    if (d.nred > 0 && on < 65536 && red_total >= 64) {
        // Few outputs, each the sum of many values: a thread per output would walk them alone (the row sums of
        // 4096 x 4096 took 1.2 ms, [32, 12, 512, 512] down to [32, 1, 1, 512] 5 ms, 8 rows of a million 250 ms).
        // One reduced axis after the other instead, longest first, each through k_reduce_dim's forms.
        int64_t cur[MNI_MAX_DIMS];
        int order[MNI_MAX_DIMS];
        for (int k = 0; k < gnd; ++k) cur[k] = gshape[k];
        for (int i = 0; i < d.nred; ++i) order[i] = d.red_dim[i];
        for (int i = 1; i < d.nred; ++i)
            for (int j = i; j > 0 && gshape[order[j]] > gshape[order[j - 1]]; --j) { const int t = order[j]; order[j] = order[j - 1]; order[j - 1] = t; }
        const float *src = g;
        void *held = nullptr;
        for (int i = 0; i < d.nred; ++i) {
            const int k = order[i];
            int64_t outer = 1, inner = 1;
            for (int q = 0; q < k; ++q) outer *= cur[q];
            for (int q = k + 1; q < gnd; ++q) inner *= cur[q];
            void *tmp = nullptr;
            float *dst = out;
            if (i + 1 < d.nred) {
                const int rc0 = dev_alloc(&tmp, (size_t)(outer * inner) * sizeof(float));
                if (rc0 != MNI_OK) { if (held) dev_free(held); return rc0; }
                dst = (float *)tmp;
            }
            const int rc = k_reduce_dim(dst, src, outer, cur[k], inner, 1.0f);
            if (held) dev_free(held);
            held = tmp;
            if (rc != MNI_OK) { if (held) dev_free(held); return rc; }
            src = dst;
            cur[k] = 1;
        }
        return MNI_OK;
    }
    MNI_KERNEL_LAUNCH(unbroadcast_kernel, dim3(grid_for(on, TPB)), dim3(TPB), 0, ctx().stream, out, g, d, on, red_total);
    return check_launch("unbroadcast");
}

// ---- cross-entropy --------------------------------------------------------------------
// src/native/src/ops/loss.rs:24-67: per row max, exp, normalise, -ln p[target];
// loss = mean over rows.  One wavefront per row; the row losses are summed by
// a single wavefront in a fixed order.
// dl (may be null): the row's gradient for an upstream gradient of one, (p - onehot) * dl_scale, as ce_bwd_kernel
// would compute it with scale = 1 / rows.
__device__ __forceinline__ float ce_row(float *__restrict__ sm, const float *__restrict__ logits, const int32_t t,
                                        const int64_t row, const int lane, const int64_t v, float *__restrict__ dl = nullptr,
                                        const float dl_scale = 0.f) {
    const float *x = logits + row * v;
    float *p = sm + row * v;
    float mx = -INFINITY;
    for (int64_t j = lane; j < v; j += 64) mx = fmaxf(mx, x[j]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
    for (int64_t j = lane; j < v; j += 64) {
        const float e = expf(x[j] - mx);
        p[j] = e;
        sum += e;
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    for (int64_t j = lane; j < v; j += 64) {
        const float q = p[j] / sum;
        p[j] = q;
        if (dl) dl[row * v + j] = (j == t ? q - 1.0f : q) * dl_scale;
    }
    const float e = expf(x[t] - mx);
    return -logf(e / sum);  // the row's loss (every lane holds it)
}
__global__ void ce_rows_kernel(float *__restrict__ row_loss, float *__restrict__ sm, const float *__restrict__ logits,
                               const int32_t *__restrict__ targets, int64_t n, int64_t v) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n) return;
    const float l = ce_row(sm, logits, targets[row], row, lane, v);
    if (lane == 0) row_loss[row] = l;
}
// The same with the row held in registers (NV 16-byte pieces per lane): the
// logits are read once and the probabilities written once.
template <int NV>
__device__ __forceinline__ float ce_row_cached(float *__restrict__ sm, const float *__restrict__ logits, const int32_t t,
                                               const int64_t row, const int lane, const int64_t v, float *__restrict__ dl = nullptr,
                                               const float dl_scale = 0.f) {
    const int64_t v4 = v >> 2;
    const float4 *x = reinterpret_cast<const float4 *>(logits + row * v);
    float4 *p = reinterpret_cast<float4 *>(sm + row * v);
    float4 r[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t j = lane + 64 * i;
        r[i] = j < v4 ? x[j] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < NV; ++i) mx = fmaxf(fmaxf(mx, fmaxf(r[i].x, r[i].y)), fmaxf(r[i].z, r[i].w));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        if (lane + 64 * i < v4) {
            r[i].x = expf(r[i].x - mx); r[i].y = expf(r[i].y - mx); r[i].z = expf(r[i].z - mx); r[i].w = expf(r[i].w - mx);
            sum += r[i].x; sum += r[i].y; sum += r[i].z; sum += r[i].w;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t j = lane + 64 * i;
        if (j < v4) {
            const float4 q = make_float4(r[i].x / sum, r[i].y / sum, r[i].z / sum, r[i].w / sum);
            p[j] = q;
            if (dl) {
                const int64_t c = 4 * j;
                reinterpret_cast<float4 *>(dl + row * v)[j] =
                    make_float4((c == t ? q.x - 1.0f : q.x) * dl_scale, (c + 1 == t ? q.y - 1.0f : q.y) * dl_scale,
                                (c + 2 == t ? q.z - 1.0f : q.z) * dl_scale, (c + 3 == t ? q.w - 1.0f : q.w) * dl_scale);
            }
        }
    }
    const float e = expf(logits[row * v + t] - mx);
    return -logf(e / sum);
}
template <int NV>
__global__ void ce_rows_cached_kernel(float *__restrict__ row_loss, float *__restrict__ sm, const float *__restrict__ logits,
                                      const int32_t *__restrict__ targets, int64_t n, int64_t v) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (row >= n) return;
    const float l = ce_row_cached<NV>(sm, logits, targets[row], row, lane, v);
    if (lane == 0) row_loss[row] = l;
}
// Long rows: one workgroup per row, NV 16-byte pieces per thread, maximum and sum through LDS (the four
// wavefront sums are added in wavefront order).  A wavefront per row would hold 128 registers of logits at
// 8192 classes, and a few thousand such wavefronts do not fit the chip in one round.
template <int NV>
__global__ __launch_bounds__(256) void ce_rows_wg_kernel(float *__restrict__ row_loss, float *__restrict__ sm,
                                                         const float *__restrict__ logits, const int32_t *__restrict__ targets,
                                                         int64_t n, int64_t v) {
    __shared__ float red[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t row = blockIdx.x;
    const int64_t v4 = v >> 2;
    const float4 *x = reinterpret_cast<const float4 *>(logits + row * v);
    float4 *p = reinterpret_cast<float4 *>(sm + row * v);
    float4 r[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t j = tid + 256 * i;
        r[i] = j < v4 ? x[j] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < NV; ++i) mx = fmaxf(fmaxf(mx, fmaxf(r[i].x, r[i].y)), fmaxf(r[i].z, r[i].w));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    if (lane == 0) red[0][wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        if (tid + 256 * i < v4) {
            r[i].x = expf(r[i].x - mx); r[i].y = expf(r[i].y - mx); r[i].z = expf(r[i].z - mx); r[i].w = expf(r[i].w - mx);
            sum += r[i].x; sum += r[i].y; sum += r[i].z; sum += r[i].w;
        }
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) red[1][wave] = sum;
    __syncthreads();
    sum = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t j = tid + 256 * i;
        if (j < v4) p[j] = make_float4(r[i].x / sum, r[i].y / sum, r[i].z / sum, r[i].w / sum);
    }
    if (tid == 0) {
        const int32_t t = targets[row];
        const float e = expf(logits[row * v + t] - mx);
        row_loss[row] = -logf(e / sum);
    }
}
// Rows beyond what the forms above hold in registers (a vocabulary of tens of thousands, or a row not in whole
// 16-byte pieces): a workgroup per row, three passes over the row.
__global__ __launch_bounds__(1024) void ce_rows_wide_kernel(float *__restrict__ row_loss, float *__restrict__ sm,
                                                            const float *__restrict__ logits, const int32_t *__restrict__ targets,
                                                            int64_t v, int vec) {
    __shared__ float red[32];
    const int64_t row = blockIdx.x;
    float mx, sum;
    softmax_line_workgroup(sm + row * v, logits + row * v, v, vec != 0, red, mx, sum);
    if (threadIdx.x == 0) {
        const int32_t t = targets[row];
        const float e = expf(logits[row * v + t] - mx);
        row_loss[row] = -logf(e / sum);
    }
}
__global__ void ce_mean_kernel(float *__restrict__ loss, const float *__restrict__ row_loss, int64_t n) {
    const int lane = threadIdx.x;
    float s = 0.f;
    for (int64_t i = lane; i < n; i += 64) s += row_loss[i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == 0) loss[0] = s / (float)n;
}
// A small batch in one launch: one workgroup of sixteen wavefronts, which take the rows in turn (four each at
// most) and leave the row losses in LDS; the first wavefront then adds them in ce_mean_kernel's order.  Same
// sums as the two launches.  EMBED: the targets arrive in the kernel arguments (no upload has to be queued for
// sixty-four numbers) and are written to `targets` for the backward pass.
constexpr int CE_SMALL_ROWS = 64;
constexpr int64_t CE_SMALL_VALUES = 16384;
struct CeTargets {
    int32_t t[CE_SMALL_ROWS];
};
template <int NV, bool EMBED>  // NV 0: ce_row, else ce_row_cached<NV>
__global__ __launch_bounds__(1024) void ce_small_kernel(float *__restrict__ loss, float *__restrict__ sm, const float *__restrict__ logits,
                                                        int32_t *__restrict__ targets, int n, int64_t v, float *__restrict__ dl,
                                                        const CeTargets given) {
    __shared__ float row_loss[CE_SMALL_ROWS];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int row = wave; row < n; row += 16) {
        const int32_t t = EMBED ? given.t[row] : targets[row];
        float l;
        if constexpr (NV == 0) l = ce_row(sm, logits, t, row, lane, v, dl, 1.0f / (float)n);
        else l = ce_row_cached<NV>(sm, logits, t, row, lane, v, dl, 1.0f / (float)n);
        if (lane == 0) {
            row_loss[row] = l;
            if (EMBED) targets[row] = t;
        }
    }
    __syncthreads();
    if (wave != 0) return;
    float s = 0.f;
    for (int i = lane; i < n; i += 64) s += row_loss[i];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == 0) loss[0] = s / (float)n;
}
// targets: device buffer of n values.  targets_host: null when `targets` already holds them; otherwise the
// values, which this call brings to `targets` (checked by the caller to lie in [0, v)).
// grad_for_one (may be null): n * v floats; a small batch's launch also leaves there the gradient of the logits
// for an upstream gradient of exactly one (what backward() of the loss itself asks for), and *wrote_grad says so.
int k_cross_entropy(float *loss, float *softmax, const float *logits, int32_t *targets, const int32_t *targets_host, int64_t n, int64_t v,
                    float *grad_for_one, bool *wrote_grad) {
    if (wrote_grad) *wrote_grad = false;
    MNI_TRY(ensure_init());
    if (n <= 0 || v <= 0) return set_error(MNI_ERR_INVALID, "cross_entropy: empty logits");
    const bool vec = (v % 4) == 0 && al16(logits) && al16(softmax);
    if (n <= CE_SMALL_ROWS && n * v <= CE_SMALL_VALUES && (!vec || v <= 64 * 4 * 2)) {
        CeTargets given;
        memset(&given, 0, sizeof given);
        if (targets_host) memcpy(given.t, targets_host, (size_t)n * sizeof(int32_t));
        const dim3 grid(1), block(1024);
        hipStream_t st = ctx().stream;
        float *dl = wrote_grad && (!vec || al16(grad_for_one)) ? grad_for_one : nullptr;
        if (dl) *wrote_grad = true;
        if (vec && targets_host) MNI_KERNEL_LAUNCH((ce_small_kernel<2, true>), grid, block, 0, st, loss, softmax, logits, targets, (int)n, v, dl, given);
        else if (vec) MNI_KERNEL_LAUNCH((ce_small_kernel<2, false>), grid, block, 0, st, loss, softmax, logits, targets, (int)n, v, dl, given);
        else if (targets_host) MNI_KERNEL_LAUNCH((ce_small_kernel<0, true>), grid, block, 0, st, loss, softmax, logits, targets, (int)n, v, dl, given);
        else MNI_KERNEL_LAUNCH((ce_small_kernel<0, false>), grid, block, 0, st, loss, softmax, logits, targets, (int)n, v, dl, given);
        return check_launch("ce_small");
    }
    if (targets_host) MNI_TRY(upload_small(targets, targets_host, (size_t)n * sizeof(int32_t)));
    void *rl = nullptr;
    MNI_TRY(dev_alloc(&rl, (size_t)n * sizeof(float)));
    const dim3 grid(grid_for(n, 4)), block(TPB);
    hipStream_t st = ctx().stream;
    if (vec && v <= 64 * 4 * 2)
        MNI_KERNEL_LAUNCH(ce_rows_cached_kernel<2>, grid, block, 0, st, (float *)rl, softmax, logits, targets, n, v);
    else if (vec && v <= 64 * 4 * 8)
        MNI_KERNEL_LAUNCH(ce_rows_cached_kernel<8>, grid, block, 0, st, (float *)rl, softmax, logits, targets, n, v);
    else if (vec && v <= 256 * 4 * 8 && n <= 0x7fffffffLL)
        MNI_KERNEL_LAUNCH(ce_rows_wg_kernel<8>, dim3((unsigned)n), dim3(256), 0, st, (float *)rl, softmax, logits, targets, n, v);
    else if (v >= 1024 && n <= 0x7fffffffLL)
        MNI_KERNEL_LAUNCH(ce_rows_wide_kernel, dim3((unsigned)n), dim3(v <= 16384 ? 256 : 1024), 0, st, (float *)rl, softmax, logits, targets, v, vec ? 1 : 0);
    else
        MNI_KERNEL_LAUNCH(ce_rows_kernel, grid, block, 0, st, (float *)rl, softmax, logits, targets, n, v);
    int rc = check_launch("ce_rows");
    if (rc == MNI_OK) {
        MNI_KERNEL_LAUNCH(ce_mean_kernel, dim3(1), dim3(64), 0, ctx().stream, loss, (const float *)rl, n);
        rc = check_launch("ce_mean");
    }
    dev_free(rl);
    return rc;
}
// src/native/src/ops/loss.rs:131-149: (softmax - onehot) * (grad / n)
__global__ void ce_bwd_kernel(float *__restrict__ dl, const float *__restrict__ sm, const int32_t *__restrict__ targets,
                              const float *__restrict__ grad, int64_t n, int64_t v) {
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    const float scale = grad[0] / (float)n;
    for (; idx < n * v; idx += step) {
        const int64_t row = idx / v, j = idx - row * v;
        float p = sm[idx];
        if (j == targets[row]) p -= 1.0f;
        dl[idx] = p * scale;
    }
}
// The same on 16-byte pieces, rows on the second grid axis: no division per element.
__global__ void ce_bwd4_kernel(float4 *__restrict__ dl, const float4 *__restrict__ sm, const int32_t *__restrict__ targets,
                               const float *__restrict__ grad, int64_t n, int64_t v4) {
    const float scale = grad[0] / (float)n;
    for (int64_t row = blockIdx.y; row < n; row += gridDim.y) {
        const int64_t t = targets[row];
        for (int64_t j = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; j < v4; j += (int64_t)gridDim.x * blockDim.x) {
            float4 p = sm[row * v4 + j];
            const int64_t at = t - 4 * j;  // 0 .. 3 when the target's column is in this piece
            if (at == 0) p.x -= 1.0f;
            if (at == 1) p.y -= 1.0f;
            if (at == 2) p.z -= 1.0f;
            if (at == 3) p.w -= 1.0f;
            dl[row * v4 + j] = make_float4(p.x * scale, p.y * scale, p.z * scale, p.w * scale);
        }
    }
}
int k_cross_entropy_backward(float *dlogits, const float *softmax, const int32_t *targets, const float *grad_scalar,
                             int64_t n, int64_t v) {
    MNI_TRY(ensure_init());
    if (n * v <= 0) return MNI_OK;
    if (v % 4 == 0 && al16(dlogits) && al16(softmax)) {
        const int64_t v4 = v / 4;
        const unsigned gx = (unsigned)min((int64_t)64, (v4 + TPB - 1) / TPB), gy = (unsigned)min(n, (int64_t)65535);
        MNI_KERNEL_LAUNCH(ce_bwd4_kernel, dim3(gx, gy), dim3(TPB), 0, ctx().stream, (float4 *)dlogits, (const float4 *)softmax, targets,
                           grad_scalar, n, v4);
        return check_launch("ce_backward");
    }
    MNI_KERNEL_LAUNCH(ce_bwd_kernel, dim3(grid_for(n * v, TPB * 2)), dim3(TPB), 0, ctx().stream, dlogits, softmax, targets, grad_scalar, n, v);
    return check_launch("ce_backward");
}

// ---- optimiser -----------------------------------------------------------------------
// grad_norm (src/native/src/ops/optimizer.rs:126-138): f64 accumulation.
__global__ void sumsq_kernel(double *__restrict__ part, const float *__restrict__ g, int64_t n) {
    __shared__ double sh[4];
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    double s = 0.0;
    for (; i < n; i += step) { const double v = (double)g[i]; s += v * v; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = s;
    __syncthreads();
    if (threadIdx.x == 0) part[blockIdx.x] = (sh[0] + sh[1]) + (sh[2] + sh[3]);
}
// Sum of part[0..nparts) by one workgroup of TPB threads in a fixed order; the value in thread 0 (sh: four doubles of LDS).
__device__ __forceinline__ double sum_partials(const double *part, int nparts, double *sh) {
    double s = 0.0;
    for (int p = threadIdx.x; p < nparts; p += TPB) s += part[p];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = s;
    __syncthreads();
    return (sh[0] + sh[1]) + (sh[2] + sh[3]);
}
// out[0] (+)= sum of part[0..nparts): one workgroup, fixed order
__global__ __launch_bounds__(TPB) void sumsq_final_kernel(double *__restrict__ out, const double *__restrict__ part, int nparts, int overwrite,
                                                          unsigned long long *result_word, unsigned tag) {
    __shared__ double sh[4];
    const double s = sum_partials(part, nparts, sh);
    if (threadIdx.x == 0) {
        const double total = (overwrite ? 0.0 : out[0]) + s;
        out[0] = total;
        if (result_word) post_result_word(result_word, tag, __float_as_uint((float)total));
    }
}
int sumsq_blocks(int64_t n) {
    if (n <= 0) return 0;
    int blocks = (int)grid_for(n, TPB * 8);
    return blocks > 1024 ? 1024 : blocks;
}
int k_sumsq_partials(double *part, const float *g, int64_t n) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(sumsq_kernel, dim3(sumsq_blocks(n)), dim3(TPB), 0, ctx().stream, part, g, n);
    return check_launch("sumsq");
}
int k_sumsq_finish(double *out, const double *part, int nparts, bool overwrite, unsigned long long *result_word, unsigned tag) {
    if (nparts <= 0 && !overwrite && !result_word) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(sumsq_final_kernel, dim3(1), dim3(TPB), 0, ctx().stream, out, part, nparts < 0 ? 0 : nparts, overwrite ? 1 : 0,
                       result_word, tag);
    return check_launch("sumsq_final");
}
int k_sumsq_f64(double *out, const float *g, int64_t n) {
    if (n <= 0) return MNI_OK;
    const int blocks = sumsq_blocks(n);
    void *part = nullptr;
    MNI_TRY(dev_alloc(&part, (size_t)blocks * sizeof(double)));
    int rc = k_sumsq_partials((double *)part, g, n);
    if (rc == MNI_OK) rc = k_sumsq_finish(out, (const double *)part, blocks);
    dev_free(part);
    return rc;
}

// adamw_step, cpu arm (src/native/src/ops/optimizer.rs:21-65): decoupled decay
// only when weight_decay > 0.
__global__ void adamw_kernel(float *__restrict__ p, float *__restrict__ m, float *__restrict__ v,
                             const float *__restrict__ g, int64_t n, float lr, float b1, float b2, float eps, float wd,
                             float bc1, float bc2) {
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; i < n; i += step) {
        const float gv = g[i];
        float pv = p[i];
        if (wd > 0.0f) pv *= 1.0f - lr * wd;
        const float mv = b1 * m[i] + (1.0f - b1) * gv;
        const float vv = b2 * v[i] + (1.0f - b2) * gv * gv;
        m[i] = mv;
        v[i] = vv;
        const float m_hat = mv / bc1;
        const float v_hat = vv / bc2;
        p[i] = pv - lr * m_hat / (sqrtf(v_hat) + eps);
    }
}
int k_adamw(float *p, float *m, float *v, const float *g, int64_t n, float lr, float b1, float b2, float eps, float wd,
            float bc1, float bc2) {
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(adamw_kernel, dim3(grid_for(n, TPB * 2)), dim3(TPB), 0, ctx().stream, p, m, v, g, n, lr, b1, b2, eps, wd, bc1, bc2);
    return check_launch("adamw");
}

// The same for up to MULTI_MAX tensors in one launch (a training step updates
// dozens of parameters, most of them a few hundred values long): the table
// rides in the kernel arguments, a workgroup takes MULTI_CHUNK elements of the
// tensor its index falls into.
// Sum of squares of g[lo..hi) in f64 by one workgroup of TPB threads; the value in thread 0 (sh: four doubles of LDS).
__device__ __forceinline__ double chunk_sumsq(const float *__restrict__ g, int64_t lo, int64_t hi, double *sh) {
    double sq = 0.0;
    for (int64_t i = lo + threadIdx.x; i < hi; i += TPB) { const double x = (double)g[i]; sq += x * x; }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sq += __shfl_xor(sq, off, 64);
    if ((threadIdx.x & 63) == 0) sh[threadIdx.x >> 6] = sq;
    __syncthreads();
    return (sh[0] + sh[1]) + (sh[2] + sh[3]);
}
template <bool ADAM>
__global__ void multi_tensor_kernel(const MultiTensor t, double *__restrict__ part, float lr, float b1, float b2, float eps,
                                    float wd, float bc1, float bc2) {
    int ti = 0;
    while (ti + 1 < t.count && (int)blockIdx.x >= t.block_start[ti + 1]) ++ti;
    const int64_t n = t.n[ti];
    const int64_t lo = (int64_t)((int)blockIdx.x - t.block_start[ti]) * MULTI_CHUNK;
    const int64_t hi = lo + MULTI_CHUNK < n ? lo + MULTI_CHUNK : n;
    const float *__restrict__ g = t.g[ti];
    if (ADAM) {
        float *__restrict__ p = t.p[ti], *__restrict__ m = t.m[ti], *__restrict__ v = t.v[ti];
        const bool vec = (n % 4) == 0;  // allocator blocks are 256-byte aligned; lo is a multiple of 4
        auto upd = [&](float gv, float &pv, float &mv, float &vv) {
            if (wd > 0.0f) pv *= 1.0f - lr * wd;
            mv = b1 * mv + (1.0f - b1) * gv;
            vv = b2 * vv + (1.0f - b2) * gv * gv;
            const float m_hat = mv / bc1;
            const float v_hat = vv / bc2;
            pv = pv - lr * m_hat / (sqrtf(v_hat) + eps);
        };
        if (vec) {
            for (int64_t i = lo + 4 * threadIdx.x; i < hi; i += 4 * blockDim.x) {
                const float4 g4 = *reinterpret_cast<const float4 *>(g + i);
                float4 p4 = *reinterpret_cast<float4 *>(p + i), m4 = *reinterpret_cast<float4 *>(m + i), v4 = *reinterpret_cast<float4 *>(v + i);
                upd(g4.x, p4.x, m4.x, v4.x); upd(g4.y, p4.y, m4.y, v4.y); upd(g4.z, p4.z, m4.z, v4.z); upd(g4.w, p4.w, m4.w, v4.w);
                *reinterpret_cast<float4 *>(p + i) = p4;
                *reinterpret_cast<float4 *>(m + i) = m4;
                *reinterpret_cast<float4 *>(v + i) = v4;
            }
        } else {
            for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) upd(g[i], p[i], m[i], v[i]);
        }
    } else {
        __shared__ double sh[4];
        const double sq = chunk_sumsq(g, lo, hi, sh);
        if (threadIdx.x == 0) part[blockIdx.x] = sq;
    }
}
// STEP: the same workgroup then clips (gradients scaled in place when their norm exceeds max_norm > 0, as
// clip_and_step does before its update, src/native/src/ops/optimizer.rs:224-245) and applies the AdamW update to
// every tensor of the table: a model of a few thousand parameters takes its whole optimiser step in one launch.
struct SoloStep {
    float max_norm, lr, b1, b2, eps, wd, bc1, bc2;
};
template <bool STEP>
__global__ __launch_bounds__(TPB) void sumsq_solo_kernel(const MultiTensor t, double *__restrict__ out, unsigned long long *result_word,
                                                         unsigned tag, const SoloStep a) {
    // The host waits for this kernel, so the chunks are not taken one after the other by the whole workgroup (a
    // round trip to memory each) but four at a time, one per wavefront.  A wavefront plays the four wavefronts of
    // chunk_sumsq in turn -- lane l of "wavefront" w adds up elements lo + 64 w + l, + 256, ... -- so every sum
    // is formed in the order of the multi-launch form: same value.
    __shared__ double part[SUMSQ_SOLO_BLOCKS];
    __shared__ double fin[4];
    const int blocks = t.block_start[t.count];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    for (int b = wave; b < blocks; b += TPB / 64) {
        int ti = 0;
        while (ti + 1 < t.count && b >= t.block_start[ti + 1]) ++ti;
        const int64_t n = t.n[ti];
        const int64_t lo = (int64_t)(b - t.block_start[ti]) * MULTI_CHUNK;
        const int64_t hi = lo + MULTI_CHUNK < n ? lo + MULTI_CHUNK : n;
        const float *__restrict__ g = t.g[ti];
        double s[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            double v = 0.0;
            for (int64_t i = lo + 64 * w + lane; i < hi; i += TPB) { const double x = (double)g[i]; v += x * x; }
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
            s[w] = v;
        }
        if (lane == 0) part[b] = (s[0] + s[1]) + (s[2] + s[3]);
    }
    __syncthreads();
    const double total = sum_partials(part, blocks, fin);
    if (threadIdx.x == 0) {
        out[0] = total;
        if (result_word) post_result_word(result_word, tag, __float_as_uint((float)total));
    }
    if (!STEP) return;
    const float norm = sqrtf((float)total);  // (every thread holds the total)
    const bool clip = a.max_norm > 0.0f && norm > a.max_norm;
    const float scale = clip ? a.max_norm / norm : 1.0f;
    for (int ti = 0; ti < t.count; ++ti) {
        float *__restrict__ p = t.p[ti], *__restrict__ m = t.m[ti], *__restrict__ v = t.v[ti];
        float *g = const_cast<float *>(t.g[ti]);
        const int64_t n = t.n[ti];
        for (int64_t i = threadIdx.x; i < n; i += TPB) {
            float gv = g[i];
            if (clip) { gv *= scale; g[i] = gv; }
            float pv = p[i];
            if (a.wd > 0.0f) pv *= 1.0f - a.lr * a.wd;
            const float mv = a.b1 * m[i] + (1.0f - a.b1) * gv;
            const float vv = a.b2 * v[i] + (1.0f - a.b2) * gv * gv;
            m[i] = mv;
            v[i] = vv;
            const float m_hat = mv / a.bc1;
            const float v_hat = vv / a.bc2;
            p[i] = pv - a.lr * m_hat / (sqrtf(v_hat) + a.eps);
        }
    }
}
int multi_tensor_blocks(int64_t n) { return (int)((n + MULTI_CHUNK - 1) / MULTI_CHUNK); }
static int multi_check(const MultiTensor &t) {
    if (t.count < 1 || t.count > MULTI_MAX) return set_error(MNI_ERR_INVALID, "multi-tensor launch: %d tensors", t.count);
    int at = 0;
    for (int i = 0; i < t.count; ++i) {
        if (t.block_start[i] != at || t.n[i] <= 0) return set_error(MNI_ERR_INVALID, "multi-tensor launch: inconsistent table");
        at += multi_tensor_blocks(t.n[i]);
    }
    if (t.block_start[t.count] != at) return set_error(MNI_ERR_INVALID, "multi-tensor launch: inconsistent table");
    return MNI_OK;
}
int k_adamw_multi(const MultiTensor &t, float lr, float b1, float b2, float eps, float wd, float bc1, float bc2) {
    MNI_TRY(ensure_init());
    MNI_TRY(multi_check(t));
    MNI_KERNEL_LAUNCH(multi_tensor_kernel<true>, dim3(t.block_start[t.count]), dim3(TPB), 0, ctx().stream, t, (double *)nullptr, lr, b1,
                       b2, eps, wd, bc1, bc2);
    return check_launch("adamw_multi");
}
int k_sumsq_solo(const MultiTensor &t, double *out, unsigned long long *result_word, unsigned tag) {
    MNI_TRY(ensure_init());
    MNI_TRY(multi_check(t));
    if (t.block_start[t.count] > SUMSQ_SOLO_BLOCKS) return set_error(MNI_ERR_INVALID, "sumsq_solo: more than %d chunks", SUMSQ_SOLO_BLOCKS);
    MNI_KERNEL_LAUNCH(sumsq_solo_kernel<false>, dim3(1), dim3(TPB), 0, ctx().stream, t, out, result_word, tag, SoloStep{});
    return check_launch("sumsq_solo");
}
int k_clip_and_step_solo(const MultiTensor &t, double *out, unsigned long long *result_word, unsigned tag, float max_norm, float lr, float b1,
                         float b2, float eps, float wd, float bc1, float bc2) {
    MNI_TRY(ensure_init());
    MNI_TRY(multi_check(t));
    if (t.block_start[t.count] > SUMSQ_SOLO_BLOCKS) return set_error(MNI_ERR_INVALID, "clip_and_step_solo: more than %d chunks", SUMSQ_SOLO_BLOCKS);
    MNI_KERNEL_LAUNCH(sumsq_solo_kernel<true>, dim3(1), dim3(TPB), 0, ctx().stream, t, out, result_word, tag,
                       SoloStep{max_norm, lr, b1, b2, eps, wd, bc1, bc2});
    return check_launch("clip_and_step_solo");
}
int k_sumsq_multi(const MultiTensor &t, double *part) {
    MNI_TRY(ensure_init());
    MNI_TRY(multi_check(t));
    MNI_KERNEL_LAUNCH(multi_tensor_kernel<false>, dim3(t.block_start[t.count]), dim3(TPB), 0, ctx().stream, t, part, 0.f, 0.f, 0.f,
                       0.f, 0.f, 0.f, 0.f);
    return check_launch("sumsq_multi");
}

}  // namespace mni

using namespace mni;

extern "C" {
int mni_rocm_strided_copy(float *dst, const float *src, const int64_t *shape, const int64_t *src_strides, int ndim) {
    MNI_API_GUARD;
    if (!dst || !src || (ndim > 0 && (!shape || !src_strides))) return set_error(MNI_ERR_INVALID, "strided_copy: null argument");
    return k_strided_copy(dst, src, shape, src_strides, ndim);
}
int mni_rocm_add_bias(float *out, const float *a, const float *bias, int64_t rows, int64_t cols) {
    MNI_API_GUARD;
    if (rows < 0 || cols < 0) return set_error(MNI_ERR_INVALID, "add_bias: negative extent");
    if (rows * cols > 0 && (!out || !a || !bias)) return set_error(MNI_ERR_INVALID, "add_bias: null argument");
    return k_add_bias(out, a, bias, rows, cols);
}
int mni_rocm_colsum(float *out, const float *a, int64_t rows, int64_t cols) {
    MNI_API_GUARD;
    if (rows < 0 || cols < 0) return set_error(MNI_ERR_INVALID, "colsum: negative extent");
    if (cols > 0 && (!out || (rows > 0 && !a))) return set_error(MNI_ERR_INVALID, "colsum: null argument");
    return k_colsum(out, a, rows, cols);
}
int mni_rocm_unbroadcast(float *out, const float *g, const int64_t *g_shape, int g_ndim, const int64_t *to_shape, int to_ndim) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    if (g_ndim < 0 || to_ndim < 0 || g_ndim > MNI_MAX_DIMS || to_ndim > g_ndim) return set_error(MNI_ERR_INVALID, "unbroadcast: bad ranks %d -> %d", g_ndim, to_ndim);
    if ((g_ndim > 0 && !g_shape) || (to_ndim > 0 && !to_shape)) return set_error(MNI_ERR_INVALID, "unbroadcast: null shape");
    int64_t gn = 1, on = 1;
    for (int k = 0; k < g_ndim; ++k) { if (g_shape[k] < 0) return set_error(MNI_ERR_INVALID, "unbroadcast: negative extent"); gn *= g_shape[k]; }
    for (int k = 0; k < to_ndim; ++k) { if (to_shape[k] < 0) return set_error(MNI_ERR_INVALID, "unbroadcast: negative extent"); on *= to_shape[k]; }
    // right-aligned: every extent of `to` is the gradient's or 1 (src/native/src/utils.rs:3-20 run backwards)
    const int off = g_ndim - to_ndim;
    bool same = true;
    for (int k = 0; k < g_ndim; ++k) {
        const int64_t ext = k < off ? 1 : to_shape[k - off];
        if (ext != g_shape[k] && ext != 1) return set_error(MNI_ERR_INVALID, "unbroadcast: shapes do not broadcast");
        same = same && ext == g_shape[k];
    }
    if (on == 0) return MNI_OK;
    if (!out || (gn > 0 && !g)) return set_error(MNI_ERR_INVALID, "unbroadcast: null argument");
    if (gn == 0) return k_fill(out, 0.0f, on);
    if (same) {
        const int64_t shape1[1] = {on}, stride1[1] = {1};
        return k_strided_copy(out, g, shape1, stride1, 1);
    }
    // Only leading dims summed away ([R.., C..] -> [C..] or [1.., C..]): the two-pass column sum.
    int lead = 0;
    while (lead < to_ndim && to_shape[lead] == 1) ++lead;
    const int core = to_ndim - lead;
    bool suffix = true;
    for (int i = 0; suffix && i < core; ++i) suffix = g_shape[g_ndim - core + i] == to_shape[lead + i];
    if (suffix) return k_colsum(out, g, gn / on, on);
    return k_unbroadcast(out, g, g_shape, g_ndim, to_shape, to_ndim);
}
int mni_rocm_axpy(float *dst, const float *src, float alpha, int64_t n) {
    MNI_API_GUARD;
    if (n < 0) return set_error(MNI_ERR_INVALID, "axpy: negative length");
    if (n > 0 && (!dst || !src)) return set_error(MNI_ERR_INVALID, "axpy: null argument");
    return k_axpy(dst, src, alpha, n);
}
int mni_rocm_fill(float *dst, float value, int64_t n) {
    MNI_API_GUARD;
    if (n < 0) return set_error(MNI_ERR_INVALID, "fill: negative length");
    if (n > 0 && !dst) return set_error(MNI_ERR_INVALID, "fill: null argument");
    return k_fill(dst, value, n);
}
}
