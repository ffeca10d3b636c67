// Short-K products of two K-contiguous operands (the "NT" form) on the MFMA
// matrix cores, the whole of K taken in one go.
//
//   C[b] (M x N) = epilogue( A[b] (M x K)  *  B[b]^T (K x N) ),   K <= 64, K % 4 == 0
//
// This is the score product of an attention layer, S = Q K^T with K^T a
// permuted view (reference call sites: src/native/src/ops/matmul.rs:54-70 on a
// view made by ops/layout.rs:112-134): thousands of output tiles, two K steps
// of the tile kernel each, 8 MB read and 32 MB written at the benchmark's
// shape.  There is no K loop to pipeline, so the tile kernel's machinery (two
// LDS stages, loads a step ahead, a barrier per step, an epilogue behind the
// last step) is all overhead here; what matters is that the stores of one part
// of the tile leave while the matrix pipe works on the next.
//
// A workgroup of 256 threads (4 wavefronts, 2 x 2) owns a 128 x 128 tile:
//   1. every thread requests its 16-byte pieces of both operand panels at once
//      (whole rows of K: a half wavefront reads contiguous memory);
//   2. the panels go to LDS "K-quad major" ([k / 4][row], one float4 per row),
//      so that one 16-byte LDS read hands a lane the four K values it feeds to
//      four consecutive MFMAs (lane = row % 32 + 32 (k / 4 % 2));
//   3. each wavefront pulls its 64 + 64 rows of operand fragments into
//      registers (the panels are dead after that and LDS is reused); steps
//      2 and 3 run in two halves, the rows of every wavefront's first block
//      first, so that its MFMAs start when half the pieces have arrived;
//   4. its four 32 x 32 blocks are computed one after the other, all of K per
//      block, and while the matrix pipe runs block b + 1 the accumulators of
//      block b go through a wavefront-private LDS patch (the MFMA layout holds
//      a column per lane; the patch turns that into 16-byte pieces along rows)
//      and out to memory as whole 128-byte lines, streaming stores.
#include "common.h"
#include "gemm_internal.h"
#include <type_traits>

namespace mni {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

static constexpr int PT = 128;          // tile side
static constexpr int PSLICE = PT + 1;   // float4 per K quad of a panel (+1: the 8 lanes of one LDS store pass hit 8 different 16-byte slots)
static constexpr int PPITCH = 36;       // floats per row of a wavefront's 32 x 32 patch

__device__ __forceinline__ float pk_gelu(float x) {
    // tanh-approximation GELU of the reference (src/native/src/ops/activation.rs:15-18)
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}
__device__ __forceinline__ float pk_pick(const f32x4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }

// NCH: chunks of 8 K values (4: K <= 32, 8: K <= 64)
template <int NCH>
__global__ __launch_bounds__(256, 2) void gemm_panel_kernel(const GemmLaunch g) {
    constexpr int KQ = 2 * NCH;                       // K quads per row
    constexpr int PER_THREAD = PT * KQ / 256;         // 16-byte pieces of one panel per thread
    __shared__ f32x4 lds[2 * KQ * PSLICE];
    f32x4 *As = lds, *Bs = lds + KQ * PSLICE;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int i = lane & 31, h = lane >> 5;

    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2:
    // renumber so that every XCD works on one contiguous run of tiles.
    int64_t pid = blockIdx.x;
    {
        const int64_t total = gridDim.x;
        const int64_t q = total >> 3, rr = total & 7;
        const int64_t x = pid & 7, ii = pid >> 3;
        pid = (x < rr ? x * (q + 1) : rr * (q + 1) + (x - rr) * q) + ii;
    }
    const int tiles = g.tiles_m * g.tiles_n;
    const int batch = (int)(pid / tiles);
    const int t = (int)(pid - (int64_t)batch * tiles);
    const int tm = t / g.tiles_n, tn = t - tm * g.tiles_n;
    const int m0 = tm * PT, n0 = tn * PT;

    // ---- 1. request both panels ---------------------------------------------------
    // piece f = tid + 256 x: row f / KQ, K quad f % KQ; rows beyond the edge re-read the last valid
    // row (their products are never stored), quads beyond K are zero
    const float *Ab = g.A + (int64_t)(batch % g.a_bcount) * g.a_bs;
    const float *Bb = g.B + (int64_t)(batch % g.b_bcount) * g.b_bs;
    const int kq = g.K >> 2;
    // The pieces are requested in two halves, rows {0..31, 64..95} of both panels first: those are the rows of
    // every wavefront's first block (rows 64 wm + 0..31 of A against rows 64 wn + 0..31 of B), whose MFMAs then
    // run while the other half is still on its way.  Piece x of a thread is row tid / KQ + (256 / KQ) order[x].
    constexpr int HALF = PER_THREAD / 2;
    constexpr int ROWS_PER_PASS = 256 / KQ;  // 16 (K <= 64) or 32 (K <= 32)
    auto piece_row = [&](int x) {
        // PER_THREAD 8: passes of 16 rows in the order 0 1 4 5 | 2 3 6 7; PER_THREAD 4: passes of 32 rows, 0 2 | 1 3
        const int pass = PER_THREAD == 8 ? ((x & 4) ? (x & 1) + 2 + ((x & 2) << 1) : (x & 1) + ((x & 2) << 1)) : ((x & 1) << 1) + (x >> 1);
        return tid / KQ + ROWS_PER_PASS * pass;
    };
    f32x4 va[PER_THREAD], vb[PER_THREAD];
#pragma unroll
    for (int x = 0; x < PER_THREAD; ++x) {
        const int row = piece_row(x), q = tid % KQ;
        const bool ok = KQ * 4 == 64 && g.K == 64 ? true : q < kq;
        const float *pa = Ab + (int64_t)min(m0 + row, g.M - 1) * g.a_rs + 4 * q;   // op(A)(m, k): a_cs == 1
        const float *pb = Bb + (int64_t)min(n0 + row, g.N - 1) * g.b_cs + 4 * q;   // op(B)(k, n): b_rs == 1
        va[x] = ok ? *reinterpret_cast<const f32x4 *>(pa) : f32x4{0.f, 0.f, 0.f, 0.f};
        vb[x] = ok ? *reinterpret_cast<const f32x4 *>(pb) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // ---- 2. the first half to LDS, and this wavefront's fragments of it ---------------------------
    // fragments: rows 64 wm + 32 a + i of A, 64 wn + 32 q + i of B
    f32x4 fa[2][NCH], fb[2][NCH];
    auto stage = [&](int half) {
#pragma unroll
        for (int x = half * HALF; x < (half + 1) * HALF; ++x) {
            const int row = piece_row(x), q = tid % KQ;
            As[q * PSLICE + row] = va[x];
            Bs[q * PSLICE + row] = vb[x];
        }
        __syncthreads();
#pragma unroll
        for (int c = 0; c < NCH; ++c) {
            fa[half][c] = As[(2 * c + h) * PSLICE + 64 * wm + 32 * half + i];
            fb[half][c] = Bs[(2 * c + h) * PSLICE + 64 * wn + 32 * half + i];
        }
    };
    stage(0);
    __builtin_amdgcn_sched_barrier(0);
    floatx16 acc[2];
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[0][e] = 0.0f;
#pragma unroll
    for (int c = 0; c < NCH; ++c)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(pk_pick(fa[0][c], j), pk_pick(fb[0][c], j), acc[0], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
    // ---- 3. the second half, behind the first block's MFMAs ------------------------------------------
    stage(1);
    __syncthreads();  // the panels are dead: LDS now holds the wavefronts' patches

    // ---- 4. block by block, stores of one block under the MFMAs of the next -------------
    float *patch = reinterpret_cast<float *>(lds) + wave * (32 * PPITCH);
    float *Cb = g.C + (int64_t)batch * g.c_bs;
    const int prow = lane >> 3, pc4 = 4 * (lane & 7);  // this lane's piece of a patch pass: row prow + 8 pass, columns pc4..+3
    const bool plain = g.epilogue == MNI_EPI_NONE && !g.accumulate;

    // Per block: 4 NCH MFMAs chained on one accumulator.  A chained MFMA cannot issue before the one
    // it depends on has gone through the pipe (64 cycles), and a wavefront issues in order, so whatever
    // else the wavefront has to do is placed in the gaps between the MFMAs of the NEXT block: the 16
    // patch writes of the block just finished, then the 4 patch reads, then the 4 global stores.
    // Two accumulators alternate.  sched_barrier pins the order.
    f32x4 pv[4];  // patch rows on their way to memory
    // lane (i, h) holds column i, rows 8 (e / 4) + 4 h + e % 4 of the block
    auto patch_write = [&](const floatx16 &d, int e) { patch[(8 * (e >> 2) + 4 * h + (e & 3)) * PPITCH + i] = d[e]; };
    auto patch_read = [&](int pass) { pv[pass] = *reinterpret_cast<const f32x4 *>(patch + (prow + 8 * pass) * PPITCH + pc4); };
    // FAST: an interior tile without epilogue or accumulation -- nothing to check, one store per pass
    // (a branch per store would also put every store into a basic block of its own, out of the
    // scheduler's sight)
    float *const fast_dst = Cb + (int64_t)(m0 + 64 * wm + prow) * g.ldc + n0 + 64 * wn + pc4;
    auto store_pass = [&](auto fast, int a, int q, int pass) {
        const f32x4 v = pv[pass];
        if (decltype(fast)::value) {
            __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(fast_dst + (int64_t)(32 * a + 8 * pass) * g.ldc + 32 * q));
            return;
        }
        const int col = n0 + 64 * wn + 32 * q + pc4;
        const int row = m0 + 64 * wm + 32 * a + prow + 8 * pass;
        if (row >= g.M || col >= g.N) return;
        float *dst = Cb + (int64_t)row * g.ldc + col;
        if (plain && col + 3 < g.N) {
            __builtin_nontemporal_store(v, reinterpret_cast<f32x4 *>(dst));
            return;
        }
        float o[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            if (col + x >= g.N) continue;
            if (g.epilogue != MNI_EPI_NONE) {
                o[x] += g.bias[col + x];
                if (g.epilogue == MNI_EPI_BIAS_RELU) o[x] = fmaxf(o[x], 0.0f);
                else if (g.epilogue == MNI_EPI_BIAS_GELU) o[x] = pk_gelu(o[x]);
            }
            if (g.accumulate) o[x] += dst[x];
            dst[x] = o[x];
        }
    };
    constexpr int NM = 4 * NCH;  // MFMAs per block (16 or 32)
    // what goes behind MFMA t of the next block (NM = 32: writes at t = 0..15, reads 18..21, stores 24..27;
    // NM = 16: a write behind every MFMA, reads and stores after the block)
    auto blocks = [&](auto fast) {
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
        const int a = blk >> 1, q = blk & 1;
        const floatx16 &done = acc[blk & 1];
        if (blk < 3) {
            floatx16 &next = acc[(blk + 1) & 1];
            const int na = (blk + 1) >> 1, nq = (blk + 1) & 1;
#pragma unroll
            for (int e = 0; e < 16; ++e) next[e] = 0.0f;
#pragma unroll
            for (int t = 0; t < NM; ++t) {
                __builtin_amdgcn_sched_barrier(0);
                next = __builtin_amdgcn_mfma_f32_32x32x2f32(pk_pick(fa[na][t >> 2], t & 3), pk_pick(fb[nq][t >> 2], t & 3), next, 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                if (t < 16) patch_write(done, t);
                if (NM == 32 && t >= 18 && t < 22) patch_read(t - 18);
                if (NM == 32 && t >= 24 && t < 28) store_pass(fast, a, q, t - 24);
            }
            __builtin_amdgcn_sched_barrier(0);
            if (NM < 32) {
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) patch_read(pass);
#pragma unroll
                for (int pass = 0; pass < 4; ++pass) store_pass(fast, a, q, pass);
            }
        } else {
#pragma unroll
            for (int e = 0; e < 16; ++e) patch_write(done, e);
#pragma unroll
            for (int pass = 0; pass < 4; ++pass) patch_read(pass);
#pragma unroll
            for (int pass = 0; pass < 4; ++pass) store_pass(fast, a, q, pass);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    };
    if (plain && m0 + PT <= g.M && n0 + PT <= g.N) blocks(std::integral_constant<bool, true>());
    else blocks(std::integral_constant<bool, false>());
}

// Shapes this form takes: both operands K-contiguous, K <= 64 in whole 16-byte pieces.
bool gemm_panel_eligible(const GemmLaunch &g, int amode, int bmode) {
    return amode == 0 && bmode == 0 && g.K > 0 && g.K <= 64 && g.K % 4 == 0;
}

// g.tiles_m / g.tiles_n must count 128 x 128 tiles.
int launch_gemm_panel(const GemmLaunch &g, int amode, int bmode) {
    if (!gemm_panel_eligible(g, amode, bmode))
        return set_error(MNI_ERR_INVALID, "sgemm: the short-K panel kernel takes two K-contiguous operands with K <= 64, K %% 4 == 0");
    if (g.tiles_m != (g.M + PT - 1) / PT || g.tiles_n != (g.N + PT - 1) / PT)
        return set_error(MNI_ERR_INVALID, "sgemm: panel kernel launched with a wrong tile count");
    const int64_t blocks = (int64_t)g.tiles_m * g.tiles_n * g.batch;
    if (blocks <= 0) return MNI_OK;
    if (blocks > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "sgemm: too many tiles (%lld)", (long long)blocks);
    const dim3 grid((unsigned)blocks), block(256);
    if (g.K <= 32) MNI_KERNEL_LAUNCH((gemm_panel_kernel<4>), grid, block, 0, ctx().stream, g);
    else MNI_KERNEL_LAUNCH((gemm_panel_kernel<8>), grid, block, 0, ctx().stream, g);
    return check_launch("gemm_panel_kernel");
}

}  // namespace mni
