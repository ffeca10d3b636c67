// Products so small that a launch is most of their cost: one thread per output
// element, a sequential loop over K.
//
//   C[b] = epilogue( op(A)[b] (M x K)  *  op(B)[b] (K x N) )
//
// The reference's README example (src/native/src/ops/matmul.rs:18-78 with
// [32, 10] x [10, 64] and [32, 64] x [64, 3], and the four backward products of
// ops/matmul.rs:199-222 on the same sizes) is made of such products: a few
// thousand outputs, K of 3 to 64.  The tile and skinny kernels are built to
// stream large operands; on these sizes they spend 4 to 13 us on set-up,
// barriers, K slices and reductions that have nothing to work on.
//
// Every output is the reference CPU arm's own sum: products rounded to fp32,
// added in k order, no fused multiply-add (ops/matmul.rs:62-69 is an i-k-j
// loop of `c += a * b`), so this kernel reproduces that arm bit for bit, for
// any strides.
#include "common.h"
#include "gemm_internal.h"

namespace mni {

static constexpr int TINY_THREADS = 256;

__device__ __forceinline__ float tiny_gelu(float x) {
    // tanh-approximation GELU of the reference (src/native/src/ops/activation.rs:15-18)
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}

// A4 / W4: op(A) / op(B) has unit stride along K and is read four K values at a time.
// idx: the output this thread computes, counted over batch, rows and columns.
template <bool A4, bool W4>
__device__ __forceinline__ void gemm_tiny_output(const GemmLaunch &g, const int64_t idx) {
#pragma clang fp contract(off)  // products are rounded before they are added: no fused multiply-add in this function
    const int64_t per = (int64_t)g.M * g.N;
    if (idx >= per * g.batch) return;
    const int b = (int)(idx / per);
    const int r = (int)(idx - (int64_t)b * per);
    const int m = r / g.N, n = r - m * g.N;
    const float *__restrict__ a = g.A + (int64_t)(b % g.a_bcount) * g.a_bs + (int64_t)m * g.a_rs;
    const float *__restrict__ w = g.B + (int64_t)(b % g.b_bcount) * g.b_bs + (int64_t)n * g.b_cs;
    float acc = 0.0f;
    // An operand whose K axis has unit stride is read four K values at a time (16-byte loads need no more than the
    // 4-byte alignment every float has): with one row per lane, every 4-byte load of it would touch as many
    // cache lines as there are lanes.
    constexpr bool a4 = A4, w4 = W4;
    const int k4 = (a4 || w4) ? g.K & ~3 : 0;
#pragma unroll 4
    for (int k = 0; k < k4; k += 4) {
        float av[4], wv[4];
        if (a4) {
            const float4 t = *reinterpret_cast<const float4 *>(a + k);
            av[0] = t.x; av[1] = t.y; av[2] = t.z; av[3] = t.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) av[j] = a[(int64_t)(k + j) * g.a_cs];
        }
        if (w4) {
            const float4 t = *reinterpret_cast<const float4 *>(w + k);
            wv[0] = t.x; wv[1] = t.y; wv[2] = t.z; wv[3] = t.w;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) wv[j] = w[(int64_t)(k + j) * g.b_rs];
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) acc = acc + av[j] * wv[j];
    }
#pragma unroll 16
    for (int k = k4; k < g.K; ++k) acc = acc + a[(int64_t)k * g.a_cs] * w[(int64_t)k * g.b_rs];
    if (g.epilogue != MNI_EPI_NONE) {
        acc += g.bias[n];
        if (g.epilogue == MNI_EPI_BIAS_RELU) acc = fmaxf(acc, 0.0f);
        else if (g.epilogue == MNI_EPI_BIAS_GELU) acc = tiny_gelu(acc);
    }
    float *dst = g.C + (int64_t)b * g.c_bs + (int64_t)m * g.ldc + n;
    *dst = g.accumulate ? acc + *dst : acc;
}
template <bool A4, bool W4>
__global__ __launch_bounds__(TINY_THREADS) void gemm_tiny_kernel(const GemmLaunch g) {
    gemm_tiny_output<A4, W4>(g, (int64_t)blockIdx.x * TINY_THREADS + threadIdx.x);
}
// Two independent products in one launch: workgroups [0, blocks0) compute the first, the rest the second.
// form: bit 0 = A4, bit 1 = W4 of each product.
// A third job rides along when asked for: the column sums of a contiguous [rows, cols] matrix, one thread per column,
// rows added in order -- the bias gradient of a Linear, utils::unbroadcast's own sum (src/native/src/utils.rs:55-64).
struct TinyPairLaunch {
    GemmLaunch g[2];
    unsigned blocks0, blocks01;  // workgroups of the first product; of both products
    int form[2];
    const float *cs_src;
    float *cs_out;
    int cs_rows, cs_cols;
};
__global__ __launch_bounds__(TINY_THREADS) void gemm_tiny_pair_kernel(const TinyPairLaunch p) {
    if (blockIdx.x >= p.blocks01) {
        const int col = (int)(blockIdx.x - p.blocks01) * TINY_THREADS + threadIdx.x;
        if (col >= p.cs_cols) return;
        const float *__restrict__ src = p.cs_src + col;
        float s = 0.0f;
        for (int r = 0; r < p.cs_rows; ++r) s += src[(int64_t)r * p.cs_cols];
        p.cs_out[col] = s;
        return;
    }
    const bool second = blockIdx.x >= p.blocks0;
    const GemmLaunch &g = second ? p.g[1] : p.g[0];
    const int64_t idx = (int64_t)(blockIdx.x - (second ? p.blocks0 : 0u)) * TINY_THREADS + threadIdx.x;
    switch (second ? p.form[1] : p.form[0]) {
        case 0: gemm_tiny_output<false, false>(g, idx); break;
        case 1: gemm_tiny_output<true, false>(g, idx); break;
        case 2: gemm_tiny_output<false, true>(g, idx); break;
        default: gemm_tiny_output<true, true>(g, idx); break;
    }
}

// Few outputs and a short K: what a launch of 256-thread workgroups computes in about the time the launch takes.
// Measured on MI355X against the tile kernel's 64 x 64 tiles (us): 32 x 64 x 10 2.6 / 5.3, 32 x 3 x 64 4.7 / 6.7,
// 64 x 64 x 64 3.3 / 5.4, 256 x 256 x 64 3.5 / 5.8, 128 x 64 x 128 4.6 / 6.6, 128 x 128 x 256 7.1 / 8.6.
// Also a large batch of products of at most 256 outputs each, which would each pad a 64 x 64 tile (us, this kernel
// against the tile kernel: 65536 x (4 x 4 x 4) 6.1 / 223, 4096 x (8 x 8 x 64) 6.2 / 27.0, 4096 x (16 x 16 x 16) 6.8 / 25.2,
// 8192 x (64 x 1 x 64) 27.7 / 62.4, 8192 x (1 x 64 x 64) 20.9 / 26.5; 1024 x (32 x 32 x 32) 10.1 / 8.6 stays with tiles).
bool gemm_tiny_eligible(const GemmLaunch &g) {
    const int64_t outputs = (int64_t)g.M * g.N * g.batch;
    if (g.epilogue > MNI_EPI_BIAS_GELU || outputs <= 0) return false;
    const int64_t k = g.K > 0 ? g.K : 1;
    // With B along K and several columns, neighbouring lanes read rows of B 4 K bytes apart: 65536 outputs and 2^22
    // multiply-adds at most, and beyond K = 128 only up to 1024 outputs (64 x 256 x 256 with B transposed 10.8 / 8.8,
    // 64 x 32 x 256 10.7 / 8.5).  With B along N
    // up to 2^18 outputs and 2^23 multiply-adds: 16384 x 16 x 16
    // 3.4 / 6.0, 784 x 128 x 64 with A transposed 4.4 / 6.0, 1024 x 256 x 32 4.4 / 5.6, 4096 x 10 x 128 6.9 / 9.6; 256 x 256 x 256 7.7 / 8.9
    // stays with tiles.
    // (rows of B of up to 64 bytes are no such matter: 4096 x 64 x 10 with B transposed 3.6 / 6.1, 16384 x 16 x 16 3.8 / 5.9)
    const bool b_along_k = g.b_rs == 1 && g.N > 1 && g.K > 16;
    // (Up to 8 rows of a K beyond 128 are the column kernel's, which slices K: 1 x 256 x 256 4.2 against 6.9 here, 4 rows 4.8 / 7.1.)
    if (g.batch == 1 && g.M <= 8 && g.K > 128 && g.N >= 64 && g.N % 4 == 0 && g.b_cs == 1) return false;
    if (b_along_k ? outputs <= (g.K <= 128 ? 65536 : 1024) && g.K <= 256 && outputs * k <= (1 << 22)
                  : outputs <= (1 << 18) && g.K <= 256 && outputs * k <= (1 << 23)) return true;
    // (With B along K and several columns, neighbouring lanes read rows of B 4 K bytes apart and the limit is 2^25:
    // 4096 x (16 x 16 x 64) with B transposed 38 / 30, 2048 x (16 x 16 x 128) 37 / 23, 4096 x (8 x 8 x 64) 11 / 28.)
    const int64_t many_limit = g.b_rs == 1 && g.N > 1 && g.M > 1 ? (1 << 25) : (1 << 27);
    if (g.batch >= 64 && (int64_t)g.M * g.N <= 256 && g.K <= 128 && outputs * k <= many_limit) return true;
    // One row per batch against a B stored K-contiguous with a short K (q . K^T of one new token per head): a thread per
    // output reads its own row of B in 16-byte pieces; 256 x (1 x 4096 x 128) 122 us against 166 through tiles,
    // 1024 x (1 x 512 x 64) 27 against 85, 32 x (1 x 8192 x 64) 15 against 45, 4 x (1 x 65536 x 64) 15 against 45,
    // 128 x (1 x 4096 x 256) 121 against 144.  Two rows up to K = 64 (256 x (2 x 4096 x 64) 82 against 104; at K = 128
    // 187 against 166, and four rows 329 against 166).
    if (g.batch < 4 || g.b_rs != 1 || g.K < 4 || outputs * k > (1LL << 28)) return false;
    return (g.M == 1 && g.K <= 256) || (g.M == 2 && g.K <= 64);
}

static int tiny_form(const GemmLaunch &g) { return (g.a_cs == 1 && g.K >= 4 ? 1 : 0) | (g.b_rs == 1 && g.K >= 4 ? 2 : 0); }
static int64_t tiny_blocks(const GemmLaunch &g) { return ((int64_t)g.M * g.N * g.batch + TINY_THREADS - 1) / TINY_THREADS; }

int launch_gemm_tiny(const GemmLaunch &g) {
    if (g.epilogue > MNI_EPI_BIAS_GELU) return set_error(MNI_ERR_INVALID, "sgemm: the tiny-product kernel has no fused GELU epilogues");
    const int64_t outputs = (int64_t)g.M * g.N * g.batch;
    if (outputs <= 0) return MNI_OK;
    const int64_t blocks = tiny_blocks(g);
    if (blocks > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "sgemm: too many outputs for the tiny-product kernel");
    const dim3 grid((unsigned)blocks), block(TINY_THREADS);
    hipStream_t st = ctx().stream;
    switch (tiny_form(g)) {
        case 3: MNI_KERNEL_LAUNCH((gemm_tiny_kernel<true, true>), grid, block, 0, st, g); break;
        case 1: MNI_KERNEL_LAUNCH((gemm_tiny_kernel<true, false>), grid, block, 0, st, g); break;
        case 2: MNI_KERNEL_LAUNCH((gemm_tiny_kernel<false, true>), grid, block, 0, st, g); break;
        default: MNI_KERNEL_LAUNCH((gemm_tiny_kernel<false, false>), grid, block, 0, st, g); break;
    }
    return check_launch("gemm_tiny_kernel");
}

// Both products must pass gemm_tiny_eligible; neither may read what the other writes.
int launch_gemm_tiny_pair(const GemmLaunch &g0, const GemmLaunch &g1, const PairColsum *colsum) {
    if (!gemm_tiny_eligible(g0) || !gemm_tiny_eligible(g1))
        return set_error(MNI_ERR_INVALID, "sgemm_pair: the tiny-product pair takes two products that each fit the tiny-product kernel");
    TinyPairLaunch p;
    p.g[0] = g0;
    p.g[1] = g1;
    p.blocks0 = (unsigned)tiny_blocks(g0);
    p.blocks01 = p.blocks0 + (unsigned)tiny_blocks(g1);
    p.form[0] = tiny_form(g0);
    p.form[1] = tiny_form(g1);
    p.cs_src = nullptr; p.cs_out = nullptr; p.cs_rows = 0; p.cs_cols = 0;
    unsigned extra = 0;
    if (colsum && colsum->rows > 0 && colsum->cols > 0) {
        p.cs_src = colsum->src; p.cs_out = colsum->out; p.cs_rows = (int)colsum->rows; p.cs_cols = (int)colsum->cols;
        extra = (unsigned)((colsum->cols + TINY_THREADS - 1) / TINY_THREADS);
    }
    const dim3 grid(p.blocks01 + extra), block(TINY_THREADS);
    MNI_KERNEL_LAUNCH(gemm_tiny_pair_kernel, grid, block, 0, ctx().stream, p);
    return check_launch("gemm_tiny_pair_kernel");
}

}  // namespace mni
