// The decode product: up to 8 rows of X against a large row-major W whose size
// is what the product costs (x[4,4096] W[4096,4096]: 64 MiB read for 134 MFLOP).
// Bound by streaming W once from HBM.  The reference has no such case: its cuda
// arm sends every shape to cuBLAS (src/native/src/ops/matmul.rs:150-173).
//
// What this form does differently from skinny_cols_kernel (gemm_skinny.hip),
// which stays for every shape this one does not take:
//  * One workgroup of 16 wavefronts per CU.  A workgroup owns a unit of 128
//    columns (512-byte pieces of W rows) and one K slice; with 256 CUs and
//    N = 4096 that is 8 slices per unit instead of 64, so an eighth of the
//    K-slice partials are written and read.  All slices of a unit run on one
//    XCD (workgroup id & 7; unit = id % units and units % 8 == 0), so the
//    partials meet in that XCD's L2.
//  * A wavefront's lanes are (column lane c = lane & 31, row lane r = lane >> 5):
//    a load instruction fetches 512 bytes of two rows, row = r + 2 wave + 32 u
//    for the u-th of its 16 loads, all requested before the first is used.
//  * X reaches the lanes through a wavefront-private piece of LDS (each
//    wavefront gathers the 32 rows it needs itself: no barrier, and the loads
//    of W are already on their way), and from 3 rows on the products run on
//    v_mfma_f32_4x4x1_16b_f32 (16 independent 4 x 4 x 1 products: block = four
//    adjacent lanes, A = x[lane & 3][k], B = one column component of the four
//    lanes, result register i = row i against the lane's own column -- the
//    accumulator layout of plain FMAs at twice their rate; 4 rows x 64 MiB is
//    1.7 us of FMA issue per SIMD, and the last of it lies after the last byte
//    has arrived).
//  * Nobody waits for anybody.  A workgroup adds its wavefronts through LDS and
//    stores its partial with the launch's tag in every piece: {x, y, z, tag} as
//    16 bytes, {w, tag} as 8.  Then, without waiting for the stores, each of
//    its summing wavefronts counts itself in at the unit's counter and asks
//    for the other slices' partials -- all in flight together.  The wavefront
//    that completes a count adds the unit up in slice order, its own partial
//    from registers; it checks the tags of what it fetched (a partial whose
//    store had not landed yet is fetched again past the L1, rare) and writes
//    the output.  After the last byte of W that is: LDS sum, one trip to the
//    L2 and back, the output store -- about 1.1 us where the flag-polling
//    reducers of skinny_cols_kernel take 2.  Sums are formed in a fixed order
//    (row lanes, wavefronts, slices), so the result does not depend on who
//    adds.  The own slot is never fetched: a load of a line with the
//    wavefront's own store still in flight took tens of microseconds.
//  * Partials live in a buffer of the library's own that nothing else ever
//    writes, so a stale piece carries an older launch's tag, never this one's.
#include "common.h"
#include "gemm_internal.h"

namespace mni {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

static constexpr int GV_THREADS = 1024, GV_WAVES = 16, GV_U = 16, GV_CL = 32, GV_UNIT_COLS = 128;
static constexpr int GV_TRIP_ROWS = 2 * GV_WAVES * GV_U;  // 512 rows of K per workgroup and trip
static constexpr int GV_SPIN_LIMIT = 1 << 14;

__device__ __forceinline__ float gv_gelu(float x) {
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}

// EPI: a bias (and activation) and / or accumulation is present (the benchmark's plain product carries neither).
// FIXED: one trip and 8 slices, known at compile time (the 4096 x 4096 weight on 256 CUs)
template <int MR, bool EPI, bool FIXED>
__global__ __launch_bounds__(GV_THREADS) void gemv_units_kernel(const GemvLaunch p) {
    constexpr int U = GV_U, CL = GV_CL, SMAX = GEMV_MAX_SLICES;
    __shared__ float xs[GV_WAVES][MR][32];
    __shared__ f32x4 red[GV_WAVES][MR * CL];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int id = blockIdx.x;
    const int unit = id % p.units, slice = id / p.units;
    const int S = FIXED ? GEMV_MAX_SLICES : p.slices;
    const int trips = FIXED ? 1 : p.trips;
    const int c = lane & (CL - 1), r = lane >> 5;

    // Everything the end of the kernel needs is fetched from the argument block and worked out now, not after the
    // last byte of W has arrived.
    const unsigned epoch = p.epoch;
    const int tl = tid < MR * CL ? tid : 0;  // summing threads: (row tl >> 5, column lane tl & 31)
    const int64_t slot = (int64_t)MR * CL;
    f32x4 *const unit_a = p.pa + (int64_t)unit * S * slot;
    f32x2 *const unit_b = p.pb + (int64_t)unit * S * slot;
    f32x4 *const my_a = unit_a + (int64_t)slice * slot + tl;
    f32x2 *const my_b = unit_b + (int64_t)slice * slot + tl;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(unit_a, 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(unit_b, 0, -1, 0x00020000);
    unsigned *const my_count = p.count + unit * GEMV_COUNTERS_PER_UNIT + wave;
    f32x4 *const my_out = reinterpret_cast<f32x4 *>(p.out + (int64_t)(tl >> 5) * p.o_rs + unit * GV_UNIT_COLS + (tl & 31) * 4);
    unsigned *const status = p.status;
    const int epilogue = EPI ? p.epilogue : (int)MNI_EPI_NONE;
    asm volatile("" ::"v"(my_a), "v"(my_b), "s"(my_count), "v"(my_out), "s"(epoch), "s"(status));
    // The first slice's partial carries the bias and, when only a sum follows, the old output of an accumulating call.
    f32x4 extra = {0.f, 0.f, 0.f, 0.f};
    if (EPI && slice == 0 && tid < MR * CL) {
        if (epilogue != MNI_EPI_NONE) extra = *reinterpret_cast<const f32x4 *>(p.bias + unit * GV_UNIT_COLS + (tl & 31) * 4);
        if (p.accumulate) extra += *my_out;
    }

    constexpr int SETS = (MR + 3) / 4;
    f32x4 acc[MR];
    f32x4 cacc[SETS][4];
#pragma unroll
    for (int i = 0; i < MR; ++i) acc[i] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int st = 0; st < SETS; ++st)
#pragma unroll
        for (int cp = 0; cp < 4; ++cp) cacc[st][cp] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int64_t w_rs = p.w_rs;
    const int rows_per_slice = trips * GV_TRIP_ROWS;
    const float *__restrict__ Wc = p.W + ((int64_t)slice * rows_per_slice + r + 2 * wave) * w_rs + unit * GV_UNIT_COLS + c * 4;
    // lane j < 32 gathers the row of X that sits at position j = 16 r + u of this wavefront's 32 rows; lanes 0-31
    // take the rows i = 0, 2, ... of X, lanes 32-63 the rows i = 1, 3, ...
    const int gj = lane & 31;
    const float *__restrict__ xp = p.X + (int64_t)slice * rows_per_slice + (gj >> 4) + 2 * wave + 32 * (gj & 15);
    for (int trip = 0; trip < trips; ++trip) {
        float xg[(MR + 1) / 2];
#pragma unroll
        for (int h = 0; h < (MR + 1) / 2; ++h) {
            const int i = 2 * h + (lane >> 5);
            xg[h] = i < MR ? xp[(int64_t)i * p.x_rs] : 0.f;
        }
        __builtin_amdgcn_sched_barrier(0);
        f32x4 w[U];
#pragma unroll
        for (int u = 0; u < U; ++u) w[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(Wc + (int64_t)u * 32 * w_rs));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int h = 0; h < (MR + 1) / 2; ++h) {
            const int i = 2 * h + (lane >> 5);
            if (i < MR) xs[wave][i][gj] = xg[h];
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // same wavefront: its LDS writes are done, no barrier needed
        __builtin_amdgcn_sched_barrier(0);
        if (MR <= 2) {
#pragma unroll
            for (int u4 = 0; u4 < U / 4; ++u4) {
                f32x4 xv[MR];
#pragma unroll
                for (int i = 0; i < MR; ++i) xv[i] = *reinterpret_cast<const f32x4 *>(&xs[wave][i][16 * r + 4 * u4]);
#pragma unroll
                for (int uu = 0; uu < 4; ++uu)
#pragma unroll
                    for (int i = 0; i < MR; ++i) acc[i] += xv[i][uu] * w[4 * u4 + uu];
            }
        } else {
#pragma unroll
            for (int u4 = 0; u4 < U / 4; ++u4) {
                f32x4 xa[SETS];
#pragma unroll
                for (int st = 0; st < SETS; ++st) {
                    const int i = 4 * st + (lane & 3);
                    xa[st] = *reinterpret_cast<const f32x4 *>(&xs[wave][i < MR ? i : 0][16 * r + 4 * u4]);  // (rows past MR: computed, never stored)
                }
#pragma unroll
                for (int uu = 0; uu < 4; ++uu)
#pragma unroll
                    for (int st = 0; st < SETS; ++st)
#pragma unroll
                        for (int cp = 0; cp < 4; ++cp)
                            cacc[st][cp] = __builtin_amdgcn_mfma_f32_4x4x1f32(xa[st][uu], w[4 * u4 + uu][cp], cacc[st][cp], 0, 0, 0);
            }
        }
        Wc += (int64_t)GV_TRIP_ROWS * w_rs;
        xp += GV_TRIP_ROWS;
        // (the next trip overwrites this wavefront's piece of xs: LDS operations of one wavefront complete in order)
    }
    if (MR > 2) {
#pragma unroll
        for (int i = 0; i < MR; ++i) acc[i] = f32x4{cacc[i / 4][0][i % 4], cacc[i / 4][1][i % 4], cacc[i / 4][2][i % 4], cacc[i / 4][3][i % 4]};
    }
    // the two row lanes meet, then the wavefronts through LDS
#pragma unroll
    for (int i = 0; i < MR; ++i) {
        acc[i].x += __shfl_xor(acc[i].x, 32, 64); acc[i].y += __shfl_xor(acc[i].y, 32, 64);
        acc[i].z += __shfl_xor(acc[i].z, 32, 64); acc[i].w += __shfl_xor(acc[i].w, 32, 64);
    }
    if (lane < CL) {
#pragma unroll
        for (int i = 0; i < MR; ++i) red[wave][i * CL + c] = acc[i];
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    if (tid >= MR * CL) return;

    // Lane 0 counts the wavefront in -- now, before the workgroup's sums are added up and stored: the answer takes 0.6 us,
    // the LDS sum and the stores 0.3-0.8, and whoever turns out to be the last arrival checks the tags of what it fetched
    // anyway (a partial of a workgroup that counted in earlier and has not stored yet is fetched again).  Under an exec
    // mask from inline asm: no divergent branch, so nothing waits for the answer here.
    unsigned rank = 0;
    if (S > 1) {  // (uniform over the grid)
        unsigned long long saved;
        asm volatile("s_mov_b64 %1, exec\n\ts_mov_b64 exec, 1\n\tglobal_atomic_inc %0, %2, %3, off sc0\n\ts_mov_b64 exec, %1"
                     : "=&v"(rank), "=&s"(saved)
                     : "v"(my_count), "v"(S - 1)
                     : "memory");
    }
    // all 16 wavefronts' sums at once, then added in wavefront order
    f32x4 e[GV_WAVES];
#pragma unroll
    for (int w2 = 0; w2 < GV_WAVES; ++w2) e[w2] = red[w2][tid];
    __builtin_amdgcn_sched_barrier(0);
    f32x4 t = e[0];
#pragma unroll
    for (int w2 = 1; w2 < GV_WAVES; ++w2) t += e[w2];
    if (EPI) t += extra;
    auto finish = [&](f32x4 v) {
        if (EPI) {
            if (epilogue == MNI_EPI_BIAS_RELU) v = f32x4{fmaxf(v.x, 0.f), fmaxf(v.y, 0.f), fmaxf(v.z, 0.f), fmaxf(v.w, 0.f)};
            else if (epilogue == MNI_EPI_BIAS_GELU) v = f32x4{gv_gelu(v.x), gv_gelu(v.y), gv_gelu(v.z), gv_gelu(v.w)};
        }
        *my_out = v;
    };
    if (S == 1) { finish(t); return; }  // (uniform over the grid)

    const float tag = __uint_as_float(epoch);
    *my_a = f32x4{t.x, t.y, t.z, tag};
    *my_b = f32x2{t.w, tag};
    f32x4 a[SMAX];
    f32x2 b[SMAX];
    const int other = slice + 1 < S ? slice + 1 : 0;
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
        const unsigned so = (s == slice || s >= S) ? other : s;  // (never the own slot, never past the last)
        a[s] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, tl * 16, so * (MR * CL * 16), 0));
        b[s] = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(rb, tl * 8, so * (MR * CL * 8), 0));
    }
    // Everything asked for above has to be back before the count is looked at (and the requests must not sink below
    // the branch that follows).
    static_assert(SMAX == 8, "operand list below");
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(rank), "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]), "+v"(b[0]),
                   "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7])
                 :
                 : "memory");
    rank = __builtin_amdgcn_readfirstlane(rank);
    if (rank != (unsigned)(S - 1)) return;

    bool ok = false;
    for (int spin = 0; spin < GV_SPIN_LIMIT; ++spin) {
        unsigned bad = 0;
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            const unsigned d = (__float_as_uint(a[s].w) ^ epoch) | (__float_as_uint(b[s].y) ^ epoch);
            bad |= (s == slice || s >= S) ? 0u : d;
        }
        ok = __all(bad == 0);
        if (ok) break;
        __builtin_amdgcn_s_sleep(2);
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            const unsigned so = (s == slice || s >= S) ? other : s;
            a[s] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, tl * 16, so * (MR * CL * 16), 16));  // sc1: past this CU's L1
            b[s] = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(rb, tl * 8, so * (MR * CL * 8), 16));
        }
    }
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
        const f32x4 v = s == slice ? t : f32x4{a[s].x, a[s].y, a[s].z, b[s].x};
        if (s < S) sum += v;
    }
    if (!ok) {
        // NaN into the output and a code into the status word: the next call that waits for the stream fails with it
        const float nan = __builtin_nanf("");
        sum = f32x4{nan, nan, nan, nan};
        if (lane == 0) *status = DEVICE_STATUS_GEMV_WAIT;
    }
    finish(sum);
}

bool gemv_units_plan(int rows, int cols, int K, int cus, int xcds, int *slices, int *trips) {
    if (rows < 1 || rows > 8 || xcds != 8 || cus != 256) return false;
    if (cols % GV_UNIT_COLS != 0) return false;
    const int units = cols / GV_UNIT_COLS;
    if (units % xcds != 0 || units > cus || cus % units != 0) return false;
    const int s = cus / units;  // one workgroup per CU
    if (s > GEMV_MAX_SLICES) return false;
    if (K % (s * GV_TRIP_ROWS) != 0 || K < s * GV_TRIP_ROWS) return false;
    *slices = s;
    *trips = K / (s * GV_TRIP_ROWS);
    return true;
}

size_t gemv_units_partial_slots(int rows, int cols, int slices) { return (size_t)(cols / GV_UNIT_COLS) * slices * rows * GV_CL; }

int launch_gemv_units(const GemvLaunch &p, int rows) {
    if (p.units <= 0 || p.slices < 1 || p.slices > GEMV_MAX_SLICES || p.trips < 1)
        return set_error(MNI_ERR_INVALID, "decode product: bad plan (units %d, slices %d, trips %d)", p.units, p.slices, p.trips);
    const dim3 grid((unsigned)(p.units * p.slices)), block(GV_THREADS);
    hipStream_t st = ctx().stream;
    const bool epi = p.epilogue != MNI_EPI_NONE || p.accumulate;
    const bool fixed = p.trips == 1 && p.slices == GEMV_MAX_SLICES;
    switch (rows) {
#define MNI_GV(R) \
    case R: \
        if (epi && fixed) MNI_KERNEL_LAUNCH((gemv_units_kernel<R, true, true>), grid, block, 0, st, p); \
        else if (epi) MNI_KERNEL_LAUNCH((gemv_units_kernel<R, true, false>), grid, block, 0, st, p); \
        else if (fixed) MNI_KERNEL_LAUNCH((gemv_units_kernel<R, false, true>), grid, block, 0, st, p); \
        else MNI_KERNEL_LAUNCH((gemv_units_kernel<R, false, false>), grid, block, 0, st, p); \
        break;
        MNI_GV(1) MNI_GV(2) MNI_GV(3) MNI_GV(4) MNI_GV(5) MNI_GV(6) MNI_GV(7) MNI_GV(8)
#undef MNI_GV
    default: return set_error(MNI_ERR_INVALID, "decode product takes 1 to 8 rows, got %d", rows);
    }
    return check_launch("gemv_units_kernel");
}


// ---- the same product for up to 32 rows -------------------------------------------------------------------------
// What changes against gemv_units_kernel: the accumulators.  With the 4 x 4 x 1 blocks a lane keeps rows x 4 columns
// of sums (64 registers at 16 rows, next to the 64 its loads are in flight in); v_mfma_f32_16x16x4_f32 keeps a
// 16 x 16 tile in four registers.  Lane (n = lane & 15, q = lane >> 4) loads 16 bytes of W: row q of the instruction's
// four, columns 4 n .. 4 n + 3 of the unit's 64 -- 256 contiguous bytes of each of four consecutive rows -- and MFMA j
// takes component j (lane n stands for column 4 n + j; the result's columns are permuted the same way: register v of
// accumulators 0..3 is four adjacent columns of row 4 q + v).  A unit is 64 columns, so there are twice the units and
// half the K slices of the 8-row form; a wavefront owns 64 consecutive rows of K per trip (16 loads of four rows),
// a workgroup 1024.  X for those rows (16 or 32 rows x 64 values, 256 contiguous bytes per row) is loaded straight into
// a wavefront-private piece of LDS, and read from there one value per lane and load as the A operand (row n, K row q);
// with 17 to 32 rows every load of W is multiplied with two sets of 16 rows (eight MFMAs instead of four).  From the
// LDS sum across the 16 wavefronts on -- 256 summing threads per set, tagged partial sums, counting in, the last
// arrival adds -- the code is the 8-row form's.
static constexpr int GW_UNIT_COLS = 64, GW_WAVE_ROWS = 4 * GV_U, GW_TRIP_ROWS = GV_WAVES * GW_WAVE_ROWS;  // 64 rows per wavefront, 1024 per trip
static constexpr int GW_PIECES = 16 * 16;  // 16-byte pieces of a 16 x 64 tile
// pitch of X (floats) up to which the byte offsets of its buffer loads, 124 x_rs + 240 at most, stay below 2^31
static constexpr int GW_MAX_X_PITCH = 1 << 24;

// SETS: sets of 16 rows (1: up to 16 rows, 2: up to 32 -- the same loads of W multiplied with two sets of rows of X)
template <int SETS, bool EPI>
__global__ __launch_bounds__(GV_THREADS) void gemv_units16_kernel(const GemvLaunch p) {
    constexpr int U = GV_U, SMAX = GEMV_MAX_SLICES;
    constexpr int XROWS = 16 * SETS, PIECES = GW_PIECES * SETS, NCOUNT = GEMV_COUNTERS_PER_UNIT * SETS;
    constexpr int XS_BYTES = GV_WAVES * XROWS * GW_WAVE_ROWS * 4, RED_BYTES = GV_WAVES * PIECES * 16;
    static_assert(U == 16, "the wait for X below counts the loads of W behind it");
    // X during the loop, the wavefronts' tiles after it: the same piece of LDS.  A wavefront's tile is as large as its X
    // and takes its place, so no wavefront writes where another still reads.
    static_assert(XS_BYTES == RED_BYTES, "a wavefront's tile goes where its X was");
    __shared__ __attribute__((aligned(1024))) char lds[XS_BYTES];
    f32x4(*red)[PIECES] = reinterpret_cast<f32x4(*)[PIECES]>(lds);
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    float *const xs = reinterpret_cast<float *>(lds) + wave * (XROWS * GW_WAVE_ROWS);  // this wavefront's XROWS x 64 values of X
    const int id = blockIdx.x;
    const int unit = id % p.units, slice = id / p.units;
    const int S = p.slices, trips = p.trips, rows = p.rows;
    const int n = lane & 15, q = lane >> 4;

    // Everything the end of the kernel needs is fetched from the argument block and worked out now, not after the
    // last byte of W has arrived.
    const unsigned epoch = p.epoch;
    const int tl = tid < PIECES ? tid : 0;  // summing threads: (row tl >> 4, column quad tl & 15)
    const int64_t slot = PIECES;
    f32x4 *const unit_a = p.pa + (int64_t)unit * S * slot;
    f32x2 *const unit_b = p.pb + (int64_t)unit * S * slot;
    f32x4 *const my_a = unit_a + (int64_t)slice * slot + tl;
    f32x2 *const my_b = unit_b + (int64_t)slice * slot + tl;
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(unit_a, 0, -1, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(unit_b, 0, -1, 0x00020000);
    unsigned *const my_count = p.count + unit * NCOUNT + wave;
    const bool my_row = (tl >> 4) < rows;
    f32x4 *const my_out = reinterpret_cast<f32x4 *>(p.out + (int64_t)(my_row ? tl >> 4 : 0) * p.o_rs + unit * GW_UNIT_COLS + (tl & 15) * 4);
    unsigned *const status = p.status;
    const int epilogue = EPI ? p.epilogue : (int)MNI_EPI_NONE;
    // (with two sets of rows the loop takes every register: there the per-lane addresses are worked out after it)
    if (SETS == 1) asm volatile("" ::"v"(my_a), "v"(my_b), "s"(my_count), "v"(my_out), "s"(epoch), "s"(status));
    else asm volatile("" ::"s"(my_count), "s"(epoch), "s"(status));
    // The first slice's partial carries the bias and, when only a sum follows, the old output of an accumulating call.
    f32x4 extra = {0.f, 0.f, 0.f, 0.f};
    auto fetch_extra = [&]() {
        if (EPI && slice == 0 && tid < PIECES) {
            if (epilogue != MNI_EPI_NONE) extra = *reinterpret_cast<const f32x4 *>(p.bias + unit * GW_UNIT_COLS + (tl & 15) * 4);
            if (p.accumulate && my_row) extra += *my_out;
        }
    };
    if (SETS == 1) fetch_extra();

    f32x4 acc[SETS][4];
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[s][j] = f32x4{0.f, 0.f, 0.f, 0.f};
    const int64_t w_rs = p.w_rs;
    const int k0 = slice * trips * GW_TRIP_ROWS + wave * GW_WAVE_ROWS;  // this wavefront's first row of K
    // W: an address per lane for the first load and a byte step that is the same for all lanes (plain loads: the same
    // loads as buffer loads with scalar offsets cost half a microsecond more on a one-trip product, 14.5 against 14.0 us
    // at 16 x 4096 x 4096, and gain as much on 16 x 8192 x 8192, 43.3 against 43.9)
    const char *Wk = reinterpret_cast<const char *>(p.W + (int64_t)(k0 + q) * w_rs + unit * GW_UNIT_COLS + n * 4);
    // X goes from memory straight into LDS, a load instruction per four rows: lane (q, n) brings a 16-byte piece of row
    // 4 e + q and the hardware puts the wavefront's 64 pieces side by side in lane order, 256 bytes per row.  Which piece
    // of its row a lane brings is its n xor-ed with the row's number within the set: piece u of row r then sits at place
    // u ^ r, and the sixteen lanes that read the same u of sixteen rows (the A operand below) hit sixteen different groups
    // of four banks.  Rows past `rows` repeat the last one: their sums are never stored.
    const char *Xk = reinterpret_cast<const char *>(p.X + k0);
    int xoff[4 * SETS];
#pragma unroll
    for (int e = 0; e < 4 * SETS; ++e) {
        const int row = 4 * e + q;
        xoff[e] = (min(row, rows - 1) * p.x_rs + 4 * (n ^ (row & 15))) * 4;
    }
    const int a_idx = n * GW_WAVE_ROWS + q, n4 = 4 * n;  // (row n of a set, K row q of a load's four)
    for (int trip = 0; trip < trips; ++trip) {
        const __amdgpu_buffer_rsrc_t rx = __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(Xk), 0, -1, 0x00020000);
        // X goes out ahead of W: it is wanted first, and loads complete in the order of issue.  (The cast: with an element
        // of an array of template-dependent size as the argument, the host pass drops the kernel's launch stub.)
#pragma unroll
        for (int e = 0; e < 4 * SETS; ++e)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (__attribute__((address_space(3))) void *)(xs + 256 * e), 16, static_cast<int>(xoff[e]), 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        f32x4 w[U];
#pragma unroll
        for (int u = 0; u < U; ++u) w[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(Wk + (int64_t)u * 16 * w_rs));
        __builtin_amdgcn_sched_barrier(0);
        // X is in LDS when no more than the 16 loads of W are outstanding (the compiler does not know that the loads
        // into LDS and the reads below touch the same bytes)
        asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            // K row 4 u + q of this trip is value q of piece u: place u ^ n of row n
            float a[SETS];
#pragma unroll
            for (int s = 0; s < SETS; ++s) a[s] = xs[s * 16 * GW_WAVE_ROWS + a_idx + ((4 * u) ^ n4)];
#pragma unroll
            for (int s = 0; s < SETS; ++s)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[s][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[s], w[u][j], acc[s][j], 0, 0, 0);
        }
        Wk += (int64_t)GW_TRIP_ROWS * 4 * w_rs;
        Xk += GW_TRIP_ROWS * 4;
        // the next trip's X overwrites this one's: every read of it has to be back first
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
    }
    if (SETS > 1) fetch_extra();  // (back by the time the LDS sum is done)
    // register v of accumulators 0..3 is row 16 s + 4 q + v, columns 4 n .. 4 n + 3: one 16-byte piece
#pragma unroll
    for (int s = 0; s < SETS; ++s)
#pragma unroll
        for (int v = 0; v < 4; ++v) red[wave][(16 * s + 4 * q + v) * 16 + n] = f32x4{acc[s][0][v], acc[s][1][v], acc[s][2][v], acc[s][3][v]};
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    if (tid >= PIECES) return;
    // Lane 0 counts the wavefront in -- now, before the workgroup's sums are added up and stored: the answer takes 0.6 us,
    // the LDS sum and the stores 0.3-0.8, and whoever turns out to be the last arrival checks the tags of what it fetched
    // anyway (a partial of a workgroup that counted in earlier and has not stored yet is fetched again).  Under an exec
    // mask from inline asm: no divergent branch, so nothing waits for the answer here.
    unsigned rank = 0;
    if (S > 1) {  // (uniform over the grid)
        unsigned long long saved;
        asm volatile("s_mov_b64 %1, exec\n\ts_mov_b64 exec, 1\n\tglobal_atomic_inc %0, %2, %3, off sc0\n\ts_mov_b64 exec, %1"
                     : "=&v"(rank), "=&s"(saved)
                     : "v"(my_count), "v"(S - 1)
                     : "memory");
    }
    // all 16 wavefronts' sums at once, then added in wavefront order
    f32x4 e[GV_WAVES];
#pragma unroll
    for (int w2 = 0; w2 < GV_WAVES; ++w2) e[w2] = red[w2][tid];
    __builtin_amdgcn_sched_barrier(0);
    f32x4 t = e[0];
#pragma unroll
    for (int w2 = 1; w2 < GV_WAVES; ++w2) t += e[w2];
    if (EPI) t += extra;
    auto finish = [&](f32x4 v) {
        if (EPI) {
            if (epilogue == MNI_EPI_BIAS_RELU) v = f32x4{fmaxf(v.x, 0.f), fmaxf(v.y, 0.f), fmaxf(v.z, 0.f), fmaxf(v.w, 0.f)};
            else if (epilogue == MNI_EPI_BIAS_GELU) v = f32x4{gv_gelu(v.x), gv_gelu(v.y), gv_gelu(v.z), gv_gelu(v.w)};
        }
        if (my_row) *my_out = v;
    };
    if (S == 1) { finish(t); return; }  // (uniform over the grid)

    const float tag = __uint_as_float(epoch);
    *my_a = f32x4{t.x, t.y, t.z, tag};
    *my_b = f32x2{t.w, tag};
    f32x4 a[SMAX];
    f32x2 b[SMAX];
    const int other = slice + 1 < S ? slice + 1 : 0;
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
        const unsigned so = (s == slice || s >= S) ? other : s;  // (never the own slot, never past the last)
        a[s] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, tl * 16, so * (PIECES * 16), 0));
        b[s] = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(rb, tl * 8, so * (PIECES * 8), 0));
    }
    // Everything asked for above has to be back before the count is looked at (and the requests must not sink below
    // the branch that follows).
    static_assert(SMAX == 8, "operand list below");
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(rank), "+v"(a[0]), "+v"(a[1]), "+v"(a[2]), "+v"(a[3]), "+v"(a[4]), "+v"(a[5]), "+v"(a[6]), "+v"(a[7]), "+v"(b[0]),
                   "+v"(b[1]), "+v"(b[2]), "+v"(b[3]), "+v"(b[4]), "+v"(b[5]), "+v"(b[6]), "+v"(b[7])
                 :
                 : "memory");
    rank = __builtin_amdgcn_readfirstlane(rank);
    if (rank != (unsigned)(S - 1)) return;

    bool ok = false;
    for (int spin = 0; spin < GV_SPIN_LIMIT; ++spin) {
        unsigned bad = 0;
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            const unsigned d = (__float_as_uint(a[s].w) ^ epoch) | (__float_as_uint(b[s].y) ^ epoch);
            bad |= (s == slice || s >= S) ? 0u : d;
        }
        ok = __all(bad == 0);
        if (ok) break;
        __builtin_amdgcn_s_sleep(2);
#pragma unroll
        for (int s = 0; s < SMAX; ++s) {
            const unsigned so = (s == slice || s >= S) ? other : s;
            a[s] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, tl * 16, so * (PIECES * 16), 16));  // sc1: past this CU's L1
            b[s] = __builtin_bit_cast(f32x2, __builtin_amdgcn_raw_buffer_load_b64(rb, tl * 8, so * (PIECES * 8), 16));
        }
    }
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
        const f32x4 v = s == slice ? t : f32x4{a[s].x, a[s].y, a[s].z, b[s].x};
        if (s < S) sum += v;
    }
    if (!ok) {
        // NaN into the output and a code into the status word: the next call that waits for the stream fails with it
        const float nan = __builtin_nanf("");
        sum = f32x4{nan, nan, nan, nan};
        if (lane == 0) *status = DEVICE_STATUS_GEMV_WAIT;
    }
    finish(sum);
}

bool gemv_units16_pitches_ok(int64_t w_rs, int64_t x_rs) { return w_rs > 0 && w_rs <= 0x7fffffffLL && x_rs >= 0 && x_rs <= GW_MAX_X_PITCH; }

bool gemv_units16_plan(int rows, int cols, int K, int cus, int xcds, int *slices, int *trips) {
    if (rows < 1 || rows > 32 || xcds != 8 || cus != 256) return false;
    if (cols <= 0 || cols % GW_UNIT_COLS != 0) return false;
    const int units = cols / GW_UNIT_COLS;
    if (units % xcds != 0 || units > cus || cus % units != 0) return false;
    const int s = cus / units;  // one workgroup per CU
    if (s > GEMV_MAX_SLICES) return false;
    if (K < s * GW_TRIP_ROWS || K % (s * GW_TRIP_ROWS) != 0) return false;
    *slices = s;
    *trips = K / (s * GW_TRIP_ROWS);
    return true;
}

size_t gemv_units16_partial_slots(int rows, int cols, int slices) { return (size_t)(cols / GW_UNIT_COLS) * slices * GW_PIECES * (rows > 16 ? 2 : 1); }
size_t gemv_units16_counters(int rows, int cols) { return (size_t)(cols / GW_UNIT_COLS) * GEMV_COUNTERS_PER_UNIT * (rows > 16 ? 2 : 1); }

int launch_gemv_units16(const GemvLaunch &p) {
    if (p.units <= 0 || p.units % 8 != 0 || p.slices < 1 || p.slices > GEMV_MAX_SLICES || p.trips < 1 || p.rows < 1 || p.rows > 32 ||
        (int64_t)p.units * p.slices > 256 || p.w_rs < p.units * GW_UNIT_COLS || p.o_rs < p.units * GW_UNIT_COLS ||
        (p.rows > 1 && p.x_rs < p.slices * p.trips * GW_TRIP_ROWS) || p.x_rs > GW_MAX_X_PITCH || p.x_rs < 0 ||
        (p.x_rs % 4) != 0 || ((uintptr_t)p.X & 15) != 0 || ((uintptr_t)p.W & 15) != 0 || (p.w_rs % 4) != 0)
        return set_error(MNI_ERR_INVALID, "decode product, 16-row form: bad plan (units %d, slices %d, trips %d, rows %d)", p.units, p.slices, p.trips, p.rows);
    const dim3 grid((unsigned)(p.units * p.slices)), block(GV_THREADS);
    hipStream_t st = ctx().stream;
    const bool epi = p.epilogue != MNI_EPI_NONE || p.accumulate;
    if (p.rows > 16) {
        if (epi) MNI_KERNEL_LAUNCH((gemv_units16_kernel<2, true>), grid, block, 0, st, p);
        else MNI_KERNEL_LAUNCH((gemv_units16_kernel<2, false>), grid, block, 0, st, p);
    } else {
        if (epi) MNI_KERNEL_LAUNCH((gemv_units16_kernel<1, true>), grid, block, 0, st, p);
        else MNI_KERNEL_LAUNCH((gemv_units16_kernel<1, false>), grid, block, 0, st, p);
    }
    return check_launch("gemv_units16_kernel");
}

}  // namespace mni
