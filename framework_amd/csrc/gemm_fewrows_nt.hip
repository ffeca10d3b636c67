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
//   * A (the 4, 8, 16 or 32 rows of the instantiation x K: K up to 8192, 4096, 2048, 960) sits in LDS for the whole kernel, rows K + 16 floats apart (the 16-byte reads of the first
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
    __shared__ __attribute__((aligned(16))) float zeros[256];
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
    if (tid < 256) zeros[tid] = 0.0f;
    __syncthreads();

    const int ngroups = (N + 3) >> 2;
    const float *xrow = &xs[j * pitch + 4 * b];  // (as the A operand this lane is row 4 s + j of the set)
    const float *zrow = &zeros[4 * lane];
    for (int g = blockIdx.x + (int)gridDim.x * wave; g < ngroups; g += (int)gridDim.x * FN_WAVES) {
        const int col = 4 * g + j;
        const float *wp = p.W + (int64_t)min(col, N - 1) * p.w_cs + 4 * b;  // columns past N repeat the last one: never stored
        f32x4 acc[SETS];
#pragma unroll
        for (int s = 0; s < SETS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
        // No branch around a request: the compiler counts the loads in flight per path and waits for the fewest.
        // Requests beyond the last step repeat it (the lines are in the L1 by then); steps beyond it read zeros for A (a
        // select on the values would have to wait for them where they are asked for).
        f32x4 wr[FN_RING];
#pragma unroll
        for (int r = 0; r < FN_RING; ++r) wr[r] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(wp + 64 * min(r, steps - 1)));
        // A's values are asked of LDS ahead of the MFMAs that use them -- the round trip to LDS in front of every group of MFMAs is
        // what a wavefront otherwise waits out alone.  Up to 16 rows: a step ahead, two sets of registers that alternate with
        // the step's parity.  With 32 rows (eight sets of four) the registers do not reach for that.
        constexpr int HS = SETS <= 4 ? SETS : SETS / 2;  // sets per buffer
        f32x4 xa[2][HS];
        auto fetch = [&](int t, int s0, f32x4 *dst) {
            const float *src = t < steps ? xrow + 64 * t + s0 * 4 * pitch : zrow;  // (uniform choice)
            const int set_pitch = t < steps ? 4 * pitch : 0;
#pragma unroll
            for (int s = 0; s < HS; ++s) dst[s] = *reinterpret_cast<const f32x4 *>(src + s * set_pitch);
        };
        auto mfmas = [&](int r, int s0, const f32x4 *x) {
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int s = 0; s < HS; ++s) acc[s0 + s] = __builtin_amdgcn_mfma_f32_4x4x1f32(fn_pick(x[s], c), fn_pick(wr[r], c), acc[s0 + s], 0, 0, 0);
        };
        static_assert(FN_RING % 2 == 0, "the two buffers of A alternate with the step's parity");
        if (SETS <= 4) fetch(0, 0, xa[0]);
        for (int t0 = 0; t0 < steps; t0 += FN_RING) {
#pragma unroll
            for (int r = 0; r < FN_RING; ++r) {
                const int t = t0 + r;
                // (a uniform branch around the MFMAs of the steps past the last -- their operands are zeros -- made the compiler
                // spill and the 16-row product take 48 us instead of 33)
                if (SETS <= 4) {
                    fetch(t + 1, 0, xa[(r + 1) & 1]);
                    mfmas(r, 0, xa[r & 1]);
                } else {
                    // (the halves of a step alternating, as in the sliced form below, make the compiler spill here: the ring's
                    // twelve addresses are live as well)
                    fetch(t, 0, xa[0]);
                    fetch(t, HS, xa[1]);
                    mfmas(r, 0, xa[0]);
                    mfmas(r, HS, xa[1]);
                }
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
    const int rows = g.M > 16 ? 32 : g.M > 8 ? 16 : g.M > 4 ? 8 : 4;  // (rows of A the kernel's instantiation keeps in LDS)
    if ((int64_t)rows * (g.K + FN_XPAD) > FEWROWS_NT_LDS_FLOATS) return false;
    if (g.a_rs % 4 != 0 || g.b_cs % 4 != 0 || !fn_aligned16(g.A) || !fn_aligned16(g.B)) return false;
    if (g.a_rs < g.K || g.b_cs < g.K || g.ldc < g.N) return false;
    if (g.epilogue != MNI_EPI_NONE && !g.bias) return false;
    return true;
}

int launch_gemm_fewrows_nt(const GemmLaunch &g, int amode, int bmode) {
    if (!gemm_fewrows_nt_eligible(g, amode, bmode))
        return set_error(MNI_ERR_INVALID, "sgemm: the few-rows kernel for a K-contiguous B takes one product of up to 32 rows of a K-contiguous A, "
                                          "K %% 64 == 0 and at most 8192 / 4096 / 2048 / 960 for up to 4 / 8 / 16 / 32 rows, both operands 16-byte aligned with "
                                          "pitches in whole 16 bytes");
    FewNtLaunch p;
    p.X = g.A; p.W = g.B; p.out = g.C; p.bias = g.bias;
    p.M = g.M; p.N = g.N; p.K = g.K;
    p.x_rs = g.a_rs; p.w_cs = g.b_cs; p.o_rs = g.ldc;
    p.epilogue = g.epilogue; p.accumulate = g.accumulate;
    p.ws = nullptr; p.count = nullptr; p.slices = 1; p.ksteps = 0;
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

// ---- the same product with K in slices ----------------------------------------------------------------------------
// A weight of 4096 x 4096 kept [out, in] under 16 rows of dY (dX = dY W^T of a small batch, matmul.rs:199-222) has a K
// of 4096: 16 rows of it are 256 KB, more than LDS holds, and 1024 groups of four columns give the 4096 wavefronts
// of the chip one group each however K is cut.  So a workgroup takes 64 columns (a group per wavefront) and one slice
// of K -- a run of steps of 64 values, at most 16 of them (12 beyond 16 rows) -- and:
//   * A's slice goes from memory straight into LDS (wavefront w brings row w, and row w + 16 of 32: a load instruction
//     per four steps, 1 KB, which the hardware lays down in lane order, i.e. as the row lies in memory) and is waited
//     for before anybody asks for W: a CU takes requests only as fast as earlier ones are answered, and behind the first
//     wavefronts' loads of W the barrier that says "A is in LDS" would fall when most of W is in, with every MFMA of the
//     workgroup still to come.
//   * the steps are gemm_fewrows_nt_kernel's; a slice is at most RING steps long, so all of its W is requested before the
//     first MFMA and there is no loop.
//   * the slices of a column block run on one XCD (workgroup id = 8 q + XCD; q = block of eight column blocks x slice),
//     so their partial sums meet in that XCD's L2: a workgroup stores its 16 x 64 sums (column-major, 16 bytes per lane),
//     waits for the L2 to acknowledge them, and counts in at the column block's counter (atomic increment that wraps with
//     the last arrival, so the counters never need clearing).  Whoever completes the count adds the slices in slice
//     order -- wavefront = row, lane = column, every slice's value requested past the L1 before the first add -- applies
//     the epilogue and stores whole rows of 64 columns.  Nobody waits for anybody; the sum order is fixed.
static constexpr int FS_UNIT_COLS = 64, FS_UNIT_FLOATS = 16 * FS_UNIT_COLS * 2;  // (32 rows: two halves of 16 x 64)

__device__ __forceinline__ float fs_load_l2(__amdgpu_buffer_rsrc_t rsrc, int byte_offset) {
    // cache policy 16 = sc1: answered by the XCD's L2, never by this CU's L1
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, byte_offset, 0, 16));
}

template <int SETS, int RING>
__global__ __launch_bounds__(FN_THREADS) void gemm_fewrows_nt_sliced_kernel(const FewNtLaunch p) {
    __shared__ __attribute__((aligned(1024))) float xs[FEWROWS_NT_LDS_FLOATS];
    __shared__ unsigned arrived_before;
    __shared__ __attribute__((aligned(16))) float zeros[256];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int j = lane & 3, b = lane >> 2;
    const int M = p.M, N = p.N, S = p.slices;
    const int xcd = blockIdx.x & 7, q = blockIdx.x >> 3;
    if (tid < 256) zeros[tid] = 0.0f;  // (read behind the barrier below)
    const int slice = q % S, unit = (q / S) * 8 + xcd;
    const int n0 = unit * FS_UNIT_COLS;
    if (n0 >= N) return;  // (the column blocks are rounded up to eight per round of XCDs: the whole workgroup leaves)
    // K in steps of 64 values (a load instruction of W: 256 bytes of each of four rows); a slice is a run of steps, the first
    // ksteps % S slices one step longer.  (Dealt round-robin instead -- slice s the steps s, s + S, ..., so that a wavefront's
    // requests spread over whole rows of W -- the same product took 19.2 us instead of 17.5.)
    const int per = p.ksteps / S, rem = p.ksteps - per * S;
    const int steps = per + (slice < rem ? 1 : 0);
    const int k0 = 64 * (slice * per + min(slice, rem));
    const int pitch = 64 * 4 * ((per + (rem > 0 ? 1 : 0) + 3) >> 2) + FN_XPAD;  // floats between rows of A in LDS
    constexpr int kstride = 64;

    // ---- A's slice straight into LDS: a load instruction brings four steps of a row (lanes 16 i .. 16 i + 15: step 4 e + i);
    // rows past M repeat the last one and steps past the slice's last repeat it (neither is ever used)
    {
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.X + k0), 0, -1, 0x00020000);
        const int loads = (steps + 3) >> 2;
        for (int rr = wave; rr < 4 * SETS; rr += FN_WAVES) {
            const int rowoff = min(rr, M - 1) * (int)p.x_rs + 4 * (lane & 15);
            float *dst = xs + rr * pitch;
            for (int e = 0; e < loads; ++e) {
                const int voff = (rowoff + kstride * min(4 * e + (lane >> 4), steps - 1)) * 4;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (__attribute__((address_space(3))) void *)(dst + 256 * e), 16, voff, 0, 0, 0);
            }
        }
    }
    // A is waited for before anybody asks for W.  A CU takes requests only as fast as earlier ones are answered: with the
    // loads of W issued ahead of the barrier, the last wavefront sat in their issue for most of the stream (9 us of 12), the
    // barrier fell behind it and every MFMA of the workgroup came after that; with a few of them ahead, A queued behind the
    // whole chip's first requests for W and landed at 4-5 us.  Asked for alone it is there after 1-1.5 us, and from then on
    // a wavefront multiplies what has arrived while the others still wait for room to ask.
    __builtin_amdgcn_sched_barrier(0);
    const int col = n0 + 4 * wave + j;
    const float *wp = p.W + (int64_t)min(col, N - 1) * p.w_cs + k0 + 4 * b;  // columns past N repeat the last one: never stored
    asm volatile("" ::"v"(wp));
    // (the compiler does not connect the loads into LDS with the reads of that LDS below)
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // All of a slice's loads of W at once.  The CU serves its wavefronts oldest first, four at a time (one per SIMD): a group
    // sits in the issue of its loads until the groups before it have been answered, the last one for 9 of the stream's
    // 11 us.  (Eight loads in flight per lane and the next asked for behind every step, so that all sixteen wavefronts
    // would take their data in step by step, was no different in that -- the older wavefronts' next requests still go
    // first -- and left the last group with too few bytes in flight: 19.7 us against 19.1.)
    f32x4 wr[RING];
#pragma unroll
    for (int r = 0; r < RING; ++r) wr[r] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(wp + kstride * min(r, steps - 1)));
    __builtin_amdgcn_sched_barrier(0);

    f32x4 acc[SETS];
#pragma unroll
    for (int s = 0; s < SETS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};
    const float *xrow = &xs[j * pitch + 4 * b];  // (as the A operand this lane is row 4 s + j of the set)
    const float *zrow = &zeros[4 * lane];
    // A's values are asked of LDS ahead of the MFMAs that use them: alone on its SIMD for most of its steps -- the wavefronts get
    // their W one after the other -- a wavefront would otherwise wait out an LDS round trip in front of every group of MFMAs.
    // Up to 16 rows a step ahead (two sets of registers that alternate with the step's parity); with 32 rows the halves of a
    // step alternate (sets 4-7 under the MFMAs of sets 0-3, sets 0-3 of the next step under those of sets 4-7).
    constexpr int HS = SETS <= 4 ? SETS : SETS / 2;  // sets per buffer
    f32x4 xa[2][HS];
    // (steps past the slice's last read zeros for A: a select on the values would have to wait for them where they are asked for)
    auto fetch = [&](int t, int s0, f32x4 *dst) {
        const float *src = t < steps ? xrow + 64 * t + s0 * 4 * pitch : zrow;  // (uniform choice)
        const int set_pitch = t < steps ? 4 * pitch : 0;
#pragma unroll
        for (int s = 0; s < HS; ++s) dst[s] = *reinterpret_cast<const f32x4 *>(src + s * set_pitch);
    };
    auto mfmas = [&](int r, int s0, const f32x4 *x) {
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int s = 0; s < HS; ++s) acc[s0 + s] = __builtin_amdgcn_mfma_f32_4x4x1f32(fn_pick(x[s], c), fn_pick(wr[r], c), acc[s0 + s], 0, 0, 0);
    };
    fetch(0, 0, xa[0]);
    // a slice is at most RING steps long (fewrows_nt_max_steps)
#pragma unroll
    for (int r = 0; r < RING; ++r) {
        if (SETS <= 4) {
            if (r + 1 < RING) fetch(r + 1, 0, xa[(r + 1) & 1]);
            mfmas(r, 0, xa[r & 1]);
        } else {
            fetch(r, HS, xa[1]);
            mfmas(r, 0, xa[0]);
            __builtin_amdgcn_sched_barrier(0);
            if (r + 1 < RING) fetch(r + 1, 0, xa[0]);
            mfmas(r, HS, xa[1]);
        }
        __builtin_amdgcn_sched_barrier(0);  // (or every step's reads of A are hoisted to the top)
    }
    // the sixteen blocks' shares of K, added up over the lanes' block bits (every lane ends with the whole sum)
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
        for (int off = 4; off < 64; off <<= 1) {
            acc[s].x += __shfl_xor(acc[s].x, off, 64); acc[s].y += __shfl_xor(acc[s].y, off, 64);
            acc[s].z += __shfl_xor(acc[s].z, off, 64); acc[s].w += __shfl_xor(acc[s].w, off, 64);
        }
    // register i of lane (b, j) is row 4 s + i of column col; the lanes of block s store set s: rows 4 b .. 4 b + 3 of
    // the column, 16 bytes, and a wavefront's sixteen storing lanes 256 contiguous bytes per half of 16 rows
    float *const wsu = p.ws + ((int64_t)unit * S + slice) * FS_UNIT_FLOATS;
    if (b < SETS) {
        f32x4 c = acc[0];
#pragma unroll
        for (int s = 1; s < SETS; ++s) c = b == s ? acc[s] : c;
        *reinterpret_cast<f32x4 *>(wsu + (b >> 2) * (16 * FS_UNIT_COLS) + (4 * wave + j) * 16 + 4 * (b & 3)) = c;
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) arrived_before = atomicInc(p.count + unit, (unsigned)S - 1);  // wraps to 0 with the last
    __syncthreads();
    if (arrived_before != (unsigned)S - 1) return;

    const __amdgpu_buffer_rsrc_t rw = __builtin_amdgcn_make_buffer_rsrc(p.ws + (int64_t)unit * S * FS_UNIT_FLOATS, 0, -1, 0x00020000);
    const int ocol = n0 + lane;
#pragma unroll
    for (int half = 0; half < (SETS > 4 ? 2 : 1); ++half) {
        const int row = 16 * half + wave;
        if (row >= M) break;
        const int off = (half * (16 * FS_UNIT_COLS) + lane * 16 + wave) * 4;
        float sum = 0.0f;
        // four slices at a time, their loads in flight together; slices beyond the last repeat it and add nothing
        for (int s0 = 0; s0 < S; s0 += 4) {
            float v[4];
#pragma unroll
            for (int ds = 0; ds < 4; ++ds) v[ds] = fs_load_l2(rw, off + min(s0 + ds, S - 1) * (FS_UNIT_FLOATS * 4));
#pragma unroll
            for (int ds = 0; ds < 4; ++ds)
                if (s0 + ds < S) sum += v[ds];
        }
        if (ocol < N) {
            float o = sum;
            if (p.epilogue != MNI_EPI_NONE) o += p.bias[ocol];
            if (p.epilogue == MNI_EPI_BIAS_RELU) o = fmaxf(o, 0.0f);
            else if (p.epilogue == MNI_EPI_BIAS_GELU) o = fn_gelu(o);
            float *dst = p.out + (int64_t)row * p.o_rs + ocol;
            if (p.accumulate) o += *dst;
            *dst = o;
        }
    }
}

int fewrows_nt_max_steps(int rows) {
    return rows > 16 ? 12 : 16;  // (a slice's loads of W are all in flight at once, 16 bytes per lane each; LDS would hold 15 and 31 of A)
}

size_t fewrows_nt_sliced_ws_floats(int N, int slices) {
    const size_t units = 8 * (size_t)(((N + FS_UNIT_COLS - 1) / FS_UNIT_COLS + 7) / 8);
    return units * slices * FS_UNIT_FLOATS;
}

bool gemm_fewrows_nt_sliced_eligible(const GemmLaunch &g, int amode, int bmode) {
    if (amode != 0 || bmode != 0 || g.batch != 1 || g.M < 1 || g.M > 32 || g.N < 1 || g.epilogue > MNI_EPI_BIAS_GELU) return false;
    if (g.K < 128 || g.K % 64 != 0) return false;
    if (g.a_rs % 4 != 0 || g.b_cs % 4 != 0 || !fn_aligned16(g.A) || !fn_aligned16(g.B)) return false;
    if (g.a_rs < g.K || g.b_cs < g.K || g.ldc < g.N) return false;
    if ((int64_t)g.M * g.a_rs * 4 >= 0x7fffffffLL) return false;  // (A's rows are addressed with 32-bit byte offsets)
    if (g.epilogue != MNI_EPI_NONE && !g.bias) return false;
    return true;
}

int launch_gemm_fewrows_nt_sliced(const GemmLaunch &g, int amode, int bmode, int slices, float *ws, unsigned *count) {
    const int ksteps = g.K / 64;
    if (!gemm_fewrows_nt_sliced_eligible(g, amode, bmode) || slices < 2 || slices > FEWROWS_NT_MAX_SLICES || slices > ksteps ||
        (ksteps + slices - 1) / slices > fewrows_nt_max_steps(g.M) || !ws || !count)
        return set_error(MNI_ERR_INVALID, "sgemm: the few-rows kernel for a K-contiguous B in K slices takes one product of up to 32 rows of a K-contiguous A, "
                                          "K a multiple of 64, 2 to %d slices of at most %d values of K (%d beyond 16 rows), both operands 16-byte aligned "
                                          "with pitches in whole 16 bytes",
                         FEWROWS_NT_MAX_SLICES, fewrows_nt_max_steps(16) * 64, fewrows_nt_max_steps(32) * 64);
    FewNtLaunch p;
    p.X = g.A; p.W = g.B; p.out = g.C; p.bias = g.bias;
    p.M = g.M; p.N = g.N; p.K = g.K;
    p.x_rs = g.a_rs; p.w_cs = g.b_cs; p.o_rs = g.ldc;
    p.epilogue = g.epilogue; p.accumulate = g.accumulate;
    p.ws = ws; p.count = count; p.slices = slices;
    p.ksteps = ksteps;
    const int64_t units8 = 8 * (int64_t)(((g.N + FS_UNIT_COLS - 1) / FS_UNIT_COLS + 7) / 8);
    const int64_t wgs = units8 * slices;
    if (wgs > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "sgemm: too many workgroups (%lld)", (long long)wgs);
    hipStream_t st = ctx().stream;
    const dim3 grid((unsigned)wgs), block(FN_THREADS);
    if (g.M > 16) MNI_KERNEL_LAUNCH((gemm_fewrows_nt_sliced_kernel<8, 12>), grid, block, 0, st, p);
    else if (g.M > 8) MNI_KERNEL_LAUNCH((gemm_fewrows_nt_sliced_kernel<4, 16>), grid, block, 0, st, p);
    else if (g.M > 4) MNI_KERNEL_LAUNCH((gemm_fewrows_nt_sliced_kernel<2, 16>), grid, block, 0, st, p);
    else MNI_KERNEL_LAUNCH((gemm_fewrows_nt_sliced_kernel<1, 16>), grid, block, 0, st, p);
    return check_launch("gemm_fewrows_nt_sliced_kernel");
}

}  // namespace mni
