// A few dozen rows against a wide operand stored K-contiguous (a weight kept [out, in], a tied language-model head):
//
//   C (M x N) = epilogue( A (M x K)  *  W^T ),   W stored [N, K],   M <= 32
//
// `x.matmul(weight.transpose())` with 9 to 32 token rows (reference call site: src/native/src/ops/matmul.rs:18-78 on a
// view made by ops/layout.rs:112-134).  W is read once and is what the product costs (16 x 768 against [50304, 768]:
// 154 MB, ~25 us of HBM time, 8 us of MFMAs).  The tile kernel pads M to 64 rows, so three quarters of its MFMA time
// multiply padding, and stages W through LDS behind a barrier per K step.
//
// Here a wavefront owns 4 columns of C (4 rows of W) and all of K, so nothing is ever summed across wavefronts:
//   * v_mfma_f32_4x4x1_16b_f32 is sixteen independent 4 x 4 x 1 products, block b = lanes 4 b .. 4 b + 3: result
//     register i of lane 4 b + j is A(lane 4 b + i) * B(lane 4 b + j).  Lane (b, j) loads 16 bytes of W: row j of the
//     wavefront's four, K values 64 t + 4 b .. + 3 -- a load instruction takes 256 contiguous bytes of each of four
//     rows, eight whole cache lines (with a lane per row of W and 64 bytes per row and instruction the same product ran
//     at 3.9 TB/s, with 16 bytes per 64 at 2.2: the L1 looks up every line an instruction touches) -- and component c
//     of the load is the B operand of the MFMAs for K value 64 t + 4 b + c, one MFMA per set of four rows of A, whose
//     A operand lane (b, i) reads from LDS: row 4 s + i, the same K value.  Every block accumulates its own sixteenth
//     of K; the blocks are added up at the end of the group with four butterfly steps over the lanes' block bits.
//   * A (up to 32 rows x K) sits in LDS for the whole kernel, rows K + 16 floats apart (the 16-byte reads of the first
//     sixteen lanes -- four rows, four blocks -- then hit sixteen different bank groups).
//   * One workgroup of 16 wavefronts per CU; column group g belongs to workgroup g % workgroups, wavefront
//     g / workgroups % 16 (then round again): every CU gets the same number of groups to within one.  Twelve loads
//     per lane (K = 768: all of a group) are kept in flight; requests beyond the last repeat it.
#include "common.h"
#include "gemm_internal.h"

namespace mni {

typedef float f32x4 __attribute__((ext_vector_type(4)));

static constexpr int FN_THREADS = 1024, FN_WAVES = 16;
static constexpr int FN_RING = 12;  // loads of W in flight per lane
static constexpr int FN_XPAD = 16;  // floats between the end of a row of A in LDS and the next

__device__ __forceinline__ float fn_gelu(float x) {
    // tanh-approximation GELU of the reference (src/native/src/ops/activation.rs:15-18)
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}
__device__ __forceinline__ float fn_pick(const f32x4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }

// SETS: sets of four rows of A (1, 2, 4, 8: up to 4, 8, 16, 32 rows)
template <int SETS>
__global__ __launch_bounds__(FN_THREADS) void gemm_fewrows_nt_kernel(const FewNtLaunch p) {
    __shared__ __attribute__((aligned(16))) float xs[FEWROWS_NT_LDS_FLOATS];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 3, b = lane >> 2;
    const int K = p.K, M = p.M, N = p.N;
    const int pitch = K + FN_XPAD;  // floats between rows of A in LDS
    const int kq = K >> 2;          // 16-byte pieces per row
    const int steps = K >> 6;       // K in steps of 64: one load instruction of the wavefront

    // ---- A into LDS: piece i is row i / kq, K quad i % kq; rows past M repeat the last one (their results are never stored)
    for (int i = tid; i < SETS * 4 * kq; i += FN_THREADS) {
        const int row = i / kq, c4 = i - row * kq;
        const f32x4 v = *reinterpret_cast<const f32x4 *>(p.X + (int64_t)min(row, M - 1) * p.x_rs + 4 * c4);
        *reinterpret_cast<f32x4 *>(&xs[row * pitch + 4 * c4]) = v;
    }
    __syncthreads();

    const int ngroups = (N + 3) >> 2;
    const float *xrow = &xs[j * pitch + 4 * b];  // (as the A operand this lane is row 4 s + j of the set)
    for (int g = blockIdx.x + (int)gridDim.x * wave; g < ngroups; g += (int)gridDim.x * FN_WAVES) {
        const int col = 4 * g + j;
        const float *wp = p.W + (int64_t)min(col, N - 1) * p.w_cs + 4 * b;  // columns past N repeat the last one: never stored
        f32x4 acc[SETS];
#pragma unroll
        for (int s = 0; s < SETS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
        // No branch around a request: the compiler counts the loads in flight per path and waits for the fewest.
        // Requests beyond the last step repeat it (the lines are in the L1 by then); steps beyond it multiply zeros.
        f32x4 wr[FN_RING];
#pragma unroll
        for (int r = 0; r < FN_RING; ++r) wr[r] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(wp + 64 * min(r, steps - 1)));
        for (int t0 = 0; t0 < steps; t0 += FN_RING) {
#pragma unroll
            for (int r = 0; r < FN_RING; ++r) {
                const int t = t0 + r;
                const bool live = t < steps;
                const int tl = min(t, steps - 1);
                f32x4 xa[SETS];
#pragma unroll
                for (int s = 0; s < SETS; ++s) {
                    xa[s] = *reinterpret_cast<const f32x4 *>(xrow + s * 4 * pitch + 64 * tl);
                    if (!live) xa[s] = f32x4{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int s = 0; s < SETS; ++s) acc[s] = __builtin_amdgcn_mfma_f32_4x4x1f32(fn_pick(xa[s], c), fn_pick(wr[r], c), acc[s], 0, 0, 0);
                wr[r] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(wp + 64 * min(t + FN_RING, steps - 1)));
            }
        }
        // the sixteen blocks' shares of K, added up over the lanes' block bits (every lane ends with the whole sum)
#pragma unroll
        for (int s = 0; s < SETS; ++s)
#pragma unroll
            for (int off = 4; off < 64; off <<= 1) {
                acc[s].x += __shfl_xor(acc[s].x, off, 64); acc[s].y += __shfl_xor(acc[s].y, off, 64);
                acc[s].z += __shfl_xor(acc[s].z, off, 64); acc[s].w += __shfl_xor(acc[s].w, off, 64);
            }
        // register i of lane (b, j) is row 4 s + i of column col; the lanes of block s store set s
        if (col < N && b < SETS) {
            const float bias = p.epilogue != MNI_EPI_NONE ? p.bias[col] : 0.0f;
            f32x4 c = acc[0];
#pragma unroll
            for (int s = 1; s < SETS; ++s) c = b == s ? acc[s] : c;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = 4 * b + i;
                if (row >= M) continue;
                float o = c[i] + bias;
                if (p.epilogue == MNI_EPI_BIAS_RELU) o = fmaxf(o, 0.0f);
                else if (p.epilogue == MNI_EPI_BIAS_GELU) o = fn_gelu(o);
                float *dst = p.out + (int64_t)row * p.o_rs + col;
                if (p.accumulate) o += *dst;
                *dst = o;
            }
        }
    }
}

static bool fn_aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// Up to 32 rows of a K-contiguous A against a K-contiguous W ([N, K] with rows w_cs apart), K in whole chunks of 64
// and short enough for A to sit in LDS.
bool gemm_fewrows_nt_eligible(const GemmLaunch &g, int amode, int bmode) {
    if (amode != 0 || bmode != 0 || g.batch != 1 || g.M < 1 || g.M > 32 || g.N < 1 || g.epilogue > MNI_EPI_BIAS_GELU) return false;
    if (g.K < 64 || g.K % 64 != 0) return false;
    const int rows = g.M > 16 ? 32 : 16;
    if ((int64_t)rows * (g.K + FN_XPAD) > FEWROWS_NT_LDS_FLOATS) return false;
    if (g.a_rs % 4 != 0 || g.b_cs % 4 != 0 || !fn_aligned16(g.A) || !fn_aligned16(g.B)) return false;
    if (g.a_rs < g.K || g.b_cs < g.K || g.ldc < g.N) return false;
    if (g.epilogue != MNI_EPI_NONE && !g.bias) return false;
    return true;
}

int launch_gemm_fewrows_nt(const GemmLaunch &g, int amode, int bmode) {
    if (!gemm_fewrows_nt_eligible(g, amode, bmode))
        return set_error(MNI_ERR_INVALID, "sgemm: the few-rows kernel for a K-contiguous B takes one product of up to 32 rows of a K-contiguous A, "
                                          "K %% 64 == 0 and at most %d (%d beyond 16 rows), both operands 16-byte aligned with pitches in whole 16 bytes",
                         FEWROWS_NT_LDS_FLOATS / 16 - FN_XPAD, FEWROWS_NT_LDS_FLOATS / 32 - FN_XPAD);
    FewNtLaunch p;
    p.X = g.A; p.W = g.B; p.out = g.C; p.bias = g.bias;
    p.M = g.M; p.N = g.N; p.K = g.K;
    p.x_rs = g.a_rs; p.w_cs = g.b_cs; p.o_rs = g.ldc;
    p.epilogue = g.epilogue; p.accumulate = g.accumulate;
    const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
    const int ngroups = (g.N + 3) / 4;
    const int wgs = ngroups < cus ? ngroups : cus;
    hipStream_t st = ctx().stream;
    if (g.M > 16) MNI_KERNEL_LAUNCH((gemm_fewrows_nt_kernel<8>), dim3((unsigned)wgs), dim3(FN_THREADS), 0, st, p);
    else if (g.M > 8) MNI_KERNEL_LAUNCH((gemm_fewrows_nt_kernel<4>), dim3((unsigned)wgs), dim3(FN_THREADS), 0, st, p);
    else if (g.M > 4) MNI_KERNEL_LAUNCH((gemm_fewrows_nt_kernel<2>), dim3((unsigned)wgs), dim3(FN_THREADS), 0, st, p);
    else MNI_KERNEL_LAUNCH((gemm_fewrows_nt_kernel<1>), dim3((unsigned)wgs), dim3(FN_THREADS), 0, st, p);
    return check_launch("gemm_fewrows_nt_kernel");
}

}  // namespace mni
