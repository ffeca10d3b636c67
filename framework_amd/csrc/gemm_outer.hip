// A short K under a large output, both operands contiguous along the OUTPUT axes:
//
//   C[b] (M x N) (+)= op(A)[b] (M x K) * B[b] (K x N),   K <= 512,
//   op(A)(m, k) = A[k * a_cs + m]  (A stored [K, M]: the transposed view of an [rows, in] activation),
//   B(k, n) = B[k * b_rs + n]
//
// -- the weight gradient dW = X^T dY of a Linear layer under a small batch (reference call site:
// src/native/src/ops/matmul.rs:199-222, dB = transpose_last2(A) . dC, with K = the batch's rows).  The product
// is a sum of K outer products and costs what writing C costs (4096 x 4096: 64 MiB, ~12 us at the rate a
// plain fill reaches); the tile kernel takes 31 us for it whatever K <= 32 is: its workgroups are built around
// a long K loop (LDS staging, a barrier per step, two workgroups per CU) and here spend their lives in
// prologue and epilogue.
//
// This layout is the matrix instruction's own: lane (i, h) of v_mfma_f32_32x32x2f32 supplies A[row i][k = h]
// and B[k = h][column i], and both are contiguous along i.  So there is no LDS and no barrier:
//   * A wavefront owns 32 rows x 128 columns.  Per pair of K values it loads one float of A (row m0 + i,
//     k = 2 s + h: half a wavefront reads 128 contiguous bytes) and 16 bytes of B (row k, columns n0 + 4 i ..
//     + 3: half a wavefront reads 512 contiguous bytes) and issues four MFMAs, MFMA j taking component j of
//     B, so that in MFMA j lane i stands for column n0 + 4 i + j.
//   * The result comes out permuted the same way, which is what storing wants: element e of accumulators
//     0..3 is four adjacent columns of one row, one 16-byte store (or load, add, store when accumulating).
//   * The four wavefronts of a workgroup take four row blocks of one column group (they share B through
//     the CU's L1).  Workgroups need no LDS and ~100 registers, so several are resident per SIMD and one's
//     loads hide behind another's stores.  A small output is dealt out one wavefront per workgroup instead,
//     to reach as many CUs as it has 32 x 128 blocks.
#include "common.h"
#include "gemm_internal.h"

namespace mni {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

static constexpr int OU_ROWS = 32;    // rows per wavefront
static constexpr int OU_COLS = 128;   // columns per wavefront (and workgroup)
static constexpr int OU_WAVES = 4;    // row blocks per workgroup
static constexpr int OU_PAIRS = 4;    // pairs of K values requested together
static constexpr int OU_MAX_K = 512;

// g.tiles_n = column groups of 128, g.tiles_m = groups of 128 rows.
__global__ __launch_bounds__(256) void gemm_outer_kernel(const GemmLaunch g) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 31, h = lane >> 5;
    const int n0 = blockIdx.x * OU_COLS;
    const int m0 = (blockIdx.y * (int)(blockDim.x >> 6) + wave) * OU_ROWS;  // (workgroups of 1 or OU_WAVES wavefronts)
    const int batch = blockIdx.z;
    if (m0 >= g.M) return;  // (a whole wavefront; nothing in this kernel waits for another wavefront)

    // rows beyond M repeat the last one, columns beyond N (N % 4 == 0) the last four: neither is stored.
    // Loads are buffer loads whose per-lane part (row or column, and which of the pair's two K values) is fixed
    // and whose moving part (the K pair) is a scalar offset: the loop has no vector-ALU work between its MFMAs
    // (computing addresses and zeroing the unused half of an odd K per load made a K pair cost 470 cycles for
    // 256 of MFMAs).
    const __amdgpu_buffer_rsrc_t ar = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(g.A + (int64_t)(batch % g.a_bcount) * g.a_bs), 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t br = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float *>(g.B + (int64_t)(batch % g.b_bcount) * g.b_bs), 0, -1, 0x00020000);
    const int arow = min(m0 + i, g.M - 1), bcol = min(n0 + 4 * i, g.N - 4);
    const int a_cs = (int)g.a_cs, b_rs = (int)g.b_rs;  // (offsets fit 32 bits: checked at launch)
    const int va = (arow + h * a_cs) * 4, vb = (bcol + h * b_rs) * 4;
    const int sa = 8 * a_cs, sb = 8 * b_rs;  // bytes from one K pair to the next
    floatx16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.0f;
    auto multiply = [&](float av, const f32x4 &bv) {
        acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv.x, acc[0], 0, 0, 0);
        acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv.y, acc[1], 0, 0, 0);
        acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv.z, acc[2], 0, 0, 0);
        acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv.w, acc[3], 0, 0, 0);
    };

    // K values 2 s + h.  Whole groups of OU_PAIRS pairs first, the next group requested before the current one
    // is multiplied (a group is one round trip to memory, and a small output has no other wavefront to hide it
    // behind); then the remaining pairs, requested ahead of everything: their K indices are clamped to the last
    // row (a valid address) and what lies past an odd K is multiplied as zeros.
    const int pairs = (g.K + 1) >> 1;
    const int whole = (g.K >> 1) / OU_PAIRS;           // groups in which every K value exists
    const int rest0 = whole * OU_PAIRS;                 // first pair of the remainder
    float at[OU_PAIRS];
    f32x4 bt[OU_PAIRS];
#pragma unroll
    for (int u = 0; u < OU_PAIRS; ++u) {
        const int k = min(2 * (rest0 + u) + h, g.K - 1);
        at[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ar, (arow + k * a_cs) * 4, 0, 0));
        bt[u] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(br, (bcol + k * b_rs) * 4, 0, 0));
    }
    if (whole > 0) {
        float a[OU_PAIRS], an[OU_PAIRS];
        f32x4 b[OU_PAIRS], bn[OU_PAIRS];
        auto request = [&](int group, float (&ra)[OU_PAIRS], f32x4 (&rb)[OU_PAIRS]) {
#pragma unroll
            for (int u = 0; u < OU_PAIRS; ++u) {
                ra[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ar, va, (group * OU_PAIRS + u) * sa, 0));
                rb[u] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(br, vb, (group * OU_PAIRS + u) * sb, 0));
            }
        };
        request(0, a, b);
        for (int group = 0; group < whole; ++group) {
            request(min(group + 1, whole - 1), an, bn);  // (past the last group: the last again, unused)
#pragma unroll
            for (int u = 0; u < OU_PAIRS; ++u) multiply(a[u], b[u]);
#pragma unroll
            for (int u = 0; u < OU_PAIRS; ++u) { a[u] = an[u]; b[u] = bn[u]; }
        }
    }
#pragma unroll
    for (int u = 0; u < OU_PAIRS; ++u) {
        if (rest0 + u >= pairs) break;  // (uniform)
        const bool live = 2 * (rest0 + u) + h < g.K;
        multiply(live ? at[u] : 0.0f, live ? bt[u] : f32x4{0.f, 0.f, 0.f, 0.f});
    }

    // element e of lane (i, h): row 8 (e / 4) + 4 h + e % 4, columns n0 + 4 i + (accumulator index)
    const int col = n0 + 4 * i;
    if (col >= g.N) return;
    float *cp = g.C + (int64_t)batch * g.c_bs + col;
    if (g.accumulate) {
        f32x4 old[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int row = min(m0 + 8 * (e >> 2) + 4 * h + (e & 3), g.M - 1);
            old[e] = *reinterpret_cast<const f32x4 *>(cp + (int64_t)row * g.ldc);
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) {
            const int row = m0 + 8 * (e >> 2) + 4 * h + (e & 3);
            const f32x4 v = f32x4{acc[0][e], acc[1][e], acc[2][e], acc[3][e]} + old[e];
            if (row < g.M) *reinterpret_cast<f32x4 *>(cp + (int64_t)row * g.ldc) = v;
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const int row = m0 + 8 * (e >> 2) + 4 * h + (e & 3);
        const f32x4 v = {acc[0][e], acc[1][e], acc[2][e], acc[3][e]};
        // streaming store: C is written once and not read again here
        if (row < g.M) __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(cp + (int64_t)row * g.ldc));
    }
}

static bool ou_aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// A contiguous along M, B along N (16-byte pieces of B and C), K at most 512, no epilogue.
bool gemm_outer_eligible(const GemmLaunch &g) {
    if (g.K < 1 || g.K > OU_MAX_K || g.M < 1 || g.N < 4 || g.N % 4 != 0 || g.epilogue != MNI_EPI_NONE) return false;
    if (g.a_rs != 1 || g.b_cs != 1) return false;
    if (g.b_rs % 4 != 0 || (g.b_bcount > 1 && g.b_bs % 4 != 0) || !ou_aligned16(g.B)) return false;
    if (g.ldc % 4 != 0 || (g.batch > 1 && g.c_bs % 4 != 0) || !ou_aligned16(g.C)) return false;
    // byte offsets inside one batch of A and of B are 32-bit in the kernel
    if (g.a_cs < 0 || g.b_rs < 0 || ((int64_t)g.K * g.a_cs + g.M) * 4 >= 0x7fffffffLL || ((int64_t)g.K * g.b_rs + g.N) * 4 >= 0x7fffffffLL) return false;
    // the batch and the row blocks are grid dimensions y and z of the launch (65535 each; four row blocks per workgroup
    // once the grid is large): a product beyond that is the tile kernel's, whose grid is one-dimensional
    if (g.batch > 65535 || (g.M + OU_ROWS - 1) / OU_ROWS > 4LL * 65535) return false;
    return true;
}

int launch_gemm_outer(const GemmLaunch &g) {
    if (!gemm_outer_eligible(g))
        return set_error(MNI_ERR_INVALID, "sgemm: the short-K outer-product kernel takes an A contiguous along M and a B contiguous along N, "
                                          "K <= %d, N %% 4 == 0, B and C 16-byte aligned with row strides in whole 16 bytes, no epilogue", OU_MAX_K);
    const int64_t gx = (g.N + OU_COLS - 1) / OU_COLS, row_blocks = (g.M + OU_ROWS - 1) / OU_ROWS;
    const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
    const int waves = gx * row_blocks * g.batch <= 4LL * cus ? 1 : OU_WAVES;  // per workgroup
    const int64_t gy = (row_blocks + waves - 1) / waves;
    if (g.batch <= 0) return MNI_OK;
    if (gy > 65535 || g.batch > 65535 || gx > 0x7fffffffLL)
        return set_error(MNI_ERR_INVALID, "sgemm: too many workgroups for the outer-product kernel (%lld x %lld x %d)", (long long)gx, (long long)gy, g.batch);
    MNI_KERNEL_LAUNCH(gemm_outer_kernel, dim3((unsigned)gx, (unsigned)gy, (unsigned)g.batch), dim3(64 * waves), 0, ctx().stream, g);
    return check_launch("gemm_outer_kernel");
}

}  // namespace mni
