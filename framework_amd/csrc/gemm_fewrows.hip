// A few dozen rows against a wide, N-contiguous operand on the MFMA matrix cores:
//
//   C[b] (M x N) = epilogue( A[b] (M x K)  *  W[b] (K x N) ),   8 < M <= 32
//
// A K-contiguous, W N-contiguous -- `x.matmul(weight)` with a [in, out] weight and a batch of 9 to 32 rows
// (reference call site: src/native/src/ops/matmul.rs:18-78 through src/nn.ts:20-25), the shape of batched
// decoding.  W is read once and is what the product costs (32 rows against 4096 x 4096: 64 MiB of W, ~10 us of
// HBM time, 7 us of MFMAs).  The tile kernel spends its time elsewhere on this shape: its smallest tile pads
// M to 64 rows, stages W through LDS behind a barrier per K step and keeps one K step of loads in flight.
//
// Here W goes from memory straight into MFMA operand registers:
//   * A wavefront owns 32 rows x 128 columns and a range of K.  Lane (i, h) (i = lane % 32, h = lane / 32)
//     loads 16 bytes of W: row k, columns n0 + 4 i .. + 3 -- half a wavefront reads 512 contiguous bytes.  The
//     four values feed four v_mfma_f32_32x32x2f32, MFMA j taking component j, so in MFMA j lane i stands for
//     column n0 + 4 i + j.  The columns of the result are permuted the same way, which is exactly right for
//     storing: accumulator element e of MFMAs 0..3 is four adjacent columns of one row, one 16-byte store.
//   * K is walked in blocks of 8: lane half h takes k = 8 b + 4 h + u, u = 0..3, i.e. four loads of W (one per
//     u) and one 16-byte piece of A (row i, those four k) per block, 16 MFMAs.  Four accumulators alternate, so
//     consecutive MFMAs never depend on each other.
//   * A comes through a wavefront-private piece of LDS in chunks of 32 K values (coalesced loads, [k / 4][row]
//     in LDS: consecutive lanes read consecutive 16-byte slots), the next chunk on its way while the current
//     one is multiplied; no barrier, nobody else touches it.
//   * DEPTH blocks of W (4 DEPTH loads per lane) are requested ahead of the MFMAs that use them.
//   * The four wavefronts of a workgroup split the workgroup's K slice; at the end their partial tiles meet
//     in LDS and every wavefront adds up a quarter of the rows, in wavefront order.
//   * Workgroups = column groups x K slices.  With several slices every workgroup leaves its partial tile in
//     the workspace and counts itself in; the one that finds all others counted adds the partials in slice
//     order (whoever it is: the sum does not depend on who arrives last) and applies the epilogue.  Nobody
//     waits for anybody.  The slices of one column group all run on one XCD, so partial tiles and counter meet
//     in that XCD's L2 and no cache has to be written back or invalidated.
#include "common.h"
#include "gemm_internal.h"

namespace mni {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

static constexpr int FR_ROWS = 32;
static constexpr int FR_COLS = 128;   // columns per workgroup
// K blocks of W in flight ahead of the one being multiplied.  Time stamps per wavefront (32 x 4096 x 4096 in 8 K
// slices, one workgroup per CU): with 3 blocks ahead the loop takes 0.60 us per block, which is W arriving at
// 6.9 TB/s over the whole chip -- the memory system's rate, so more blocks in flight buy nothing (8 were tried:
// slower, for want of registers).
static constexpr int FR_DEPTH = 4;
// A reaches the MFMAs through a wavefront-private piece of LDS, a chunk of FR_CHUNK K blocks at a time, two
// chunks alternating: read straight from memory, one 16-byte piece per lane and block is 32 cache lines per
// load instruction, and that alone cost 5 us of 21 on 32 x 4096 x 4096.
static constexpr int FR_CHUNK = 4;                       // K blocks (of 8) per chunk; a multiple of FR_DEPTH
static constexpr int FR_CQ = 2 * FR_CHUNK;               // K quads per chunk
static constexpr int FR_PITCH = FR_ROWS + 1;             // 16-byte slots per K quad (+1 spreads a store pass over the banks)
static constexpr int FR_ABUF = FR_CQ * FR_PITCH;         // slots per chunk buffer
static_assert(FR_CHUNK % FR_DEPTH == 0, "the ring of W registers is indexed at compile time");

__device__ __forceinline__ float fr_gelu(float x) {
    // tanh-approximation GELU of the reference (src/native/src/ops/activation.rs:15-18)
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}
__device__ __forceinline__ f32x4 fr_load_l2(__amdgpu_buffer_rsrc_t rsrc, int byte_offset) {
    // cache policy 16 = sc1: answered by the XCD's L2, never by this CU's L1 (which may hold the line from an
    // earlier launch).  A buffer load, so that the compiler keeps track of it like of any other load and several
    // can be in flight (one round trip to L2 per load, one after the other, made the final sum take 9 us).
    return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, byte_offset, 0, 16));
}
__device__ __forceinline__ void fr_wave_sync() {
    // LDS traffic between the lanes of one wavefront.  The LDS executes a wavefront's instructions in order, so a
    // read issued after a write sees it, whichever lane wrote; all that is needed is that the compiler keeps the
    // order.  (A fence would also wait for every load of W in flight: the loop stalled at every chunk with one.)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
}
__device__ __forceinline__ float fr_pick(const f32x4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }

// g.tiles_n = column groups, g.split_k = K slices of g.k_per_slice (a multiple of 32); with split_k > 1:
// g.ws = partials [slice][batch][M][N], g.sk_flags = one counter per (batch, column group), all zero between launches.
__global__ __launch_bounds__(256, 2) void gemm_fewrows_kernel(const GemmLaunch g) {
    constexpr int RED = 16 * 4 * 64;  // floats one wavefront contributes to the workgroup's sum
    constexpr int LDS_SLOTS = 4 * 2 * FR_ABUF > RED ? 4 * 2 * FR_ABUF : RED;  // A chunks during the loop, partial tiles after it
    __shared__ f32x4 lds[LDS_SLOTS];
    __shared__ unsigned arrived_before;
    float *red = reinterpret_cast<float *>(lds);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 31, h = lane >> 5;

    // Workgroups are dealt round-robin to the XCDs (workgroup b runs on XCD b % 8), each with its own L2.  All K
    // slices of a column group run on one XCD, so that their partial tiles meet in that L2: unit u = (batch,
    // column group) belongs to XCD u % 8; the grid is padded to 8 x (units per XCD) x slices.
    const int units = g.tiles_n * g.batch;
    const int xcd = blockIdx.x & 7, ii = blockIdx.x >> 3;
    const int unit = (ii / g.split_k) * 8 + xcd, slice = ii % g.split_k;
    if (unit >= units) return;
    const int batch = unit / g.tiles_n, grp = unit - batch * g.tiles_n;
    const int n0 = grp * FR_COLS;
    const int kw = g.k_per_slice >> 2;                       // K values per wavefront (a multiple of 8)
    const int ka = slice * g.k_per_slice + wave * kw;        // this wavefront's range [ka, ka + 8 nblocks)
    const int kend = min(min(g.K, (slice + 1) * g.k_per_slice), ka + kw);
    const int nblocks = kend > ka ? (kend - ka) >> 3 : 0;

    // rows beyond M repeat the last one, columns beyond N (N % 4 == 0: a lane's four are all inside or all
    // outside) the last four inside; neither is ever stored
    // A chunk: 32 rows x FR_CQ K quads, piece p = lane + 64 t: row p / FR_CQ, quad p % FR_CQ (16 lanes read 256
    // contiguous bytes of a row); in LDS [quad][row]
    constexpr int APIECES = FR_ROWS * FR_CQ / 64;
    const int arow = lane / FR_CQ, aq = lane % FR_CQ;  // piece t: row arow + (64 / FR_CQ) t
    const float *ap = g.A + (int64_t)(batch % g.a_bcount) * g.a_bs + ka + 4 * aq;
    f32x4 *Aw = lds + wave * (2 * FR_ABUF);
    const int nq = 2 * nblocks;  // K quads of this wavefront's range
    f32x4 an[APIECES];
    auto a_request = [&](int chunk) {  // pieces of a chunk from memory into registers (quads beyond the range are zero)
        const int q = chunk * FR_CQ + aq;
#pragma unroll
        for (int t = 0; t < APIECES; ++t) {
            const int row = min(arow + (64 / FR_CQ) * t, g.M - 1);
            an[t] = q < nq ? *reinterpret_cast<const f32x4 *>(ap + (int64_t)row * g.a_rs + 4 * chunk * FR_CQ) : f32x4{0.f, 0.f, 0.f, 0.f};
        }
    };
    auto a_store = [&](int chunk) {  // ... and on into the chunk's buffer
        f32x4 *dst = Aw + (chunk & 1) * FR_ABUF;
#pragma unroll
        for (int t = 0; t < APIECES; ++t) dst[aq * FR_PITCH + arow + (64 / FR_CQ) * t] = an[t];
    };
    const int ncol = min(n0 + 4 * i, g.N - 4);
    const float *wp = g.B + (int64_t)(batch % g.b_bcount) * g.b_bs + (int64_t)(ka + 4 * h) * g.b_rs + ncol;
    const int64_t wstep = 8 * g.b_rs;
    floatx16 acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[j][e] = 0.0f;

    if (nblocks > 0) {
        // No branch inside the loop: the compiler counts the loads in flight per path and waits for the fewest, so
        // one skipped request would make every wait a wait for everything (it did: vmcnt(3..0) in front of every
        // block).  Requests beyond the range repeat the last block or chunk; blocks beyond it multiply zeros.
        const int last = nblocks - 1;
        const int nchunks = (nblocks + FR_CHUNK - 1) / FR_CHUNK;
        f32x4 wb[FR_DEPTH][4];
        a_request(0);
#pragma unroll
        for (int d = 0; d < FR_DEPTH; ++d)
#pragma unroll
            for (int u = 0; u < 4; ++u) wb[d][u] = *reinterpret_cast<const f32x4 *>(wp + min(d, last) * wstep + u * g.b_rs);
        a_store(0);
        fr_wave_sync();
        for (int c = 0; c < nchunks; ++c) {
            a_request(min(c + 1, nchunks - 1));  // on its way while this chunk is multiplied
            const f32x4 *Ac = Aw + (c & 1) * FR_ABUF;
#pragma unroll
            for (int bb = 0; bb < FR_CHUNK; ++bb) {
                const int b = c * FR_CHUNK + bb;
                const int d = bb % FR_DEPTH;
                // (blocks beyond the range: their quads of A were stored as zeros by a_request, so nothing is selected here -- a
                // select on the values would have to wait for them right behind the read)
                const f32x4 a = Ac[(2 * bb + h) * FR_PITCH + i];
#pragma unroll
                for (int u = 0; u < 4; ++u)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fr_pick(a, u), fr_pick(wb[d][u], j), acc[j], 0, 0, 0);
                const float *wn = wp + (int64_t)min(b + FR_DEPTH, last) * wstep;
#pragma unroll
                for (int u = 0; u < 4; ++u) wb[d][u] = *reinterpret_cast<const f32x4 *>(wn + u * g.b_rs);
            }
            a_store(c + 1);  // (the buffer it goes to was last read a chunk ago)
            fr_wave_sync();
        }
    }

    __syncthreads();  // every wavefront is done with its A chunks: LDS changes hands
#pragma unroll
    for (int e = 0; e < 16; ++e)
#pragma unroll
        for (int j = 0; j < 4; ++j) red[wave * RED + (e * 4 + j) * 64 + lane] = acc[j][e];
    __syncthreads();
    const int col = n0 + 4 * i;
    float *Cb = g.C + (int64_t)batch * g.c_bs;
    auto finish = [&](f32x4 v, int row, int c) {  // epilogue and store of four adjacent columns
        float *dst = Cb + (int64_t)row * g.ldc + c;
        if (g.epilogue != MNI_EPI_NONE) {
            const f32x4 bv = *reinterpret_cast<const f32x4 *>(g.bias + c);
            v += bv;
            if (g.epilogue == MNI_EPI_BIAS_RELU) v = f32x4{fmaxf(v.x, 0.0f), fmaxf(v.y, 0.0f), fmaxf(v.z, 0.0f), fmaxf(v.w, 0.0f)};
            else if (g.epilogue == MNI_EPI_BIAS_GELU) v = f32x4{fr_gelu(v.x), fr_gelu(v.y), fr_gelu(v.z), fr_gelu(v.w)};
        }
        if (g.accumulate) v += *reinterpret_cast<const f32x4 *>(dst);
        *reinterpret_cast<f32x4 *>(dst) = v;
    };
#pragma unroll
    for (int ee = 0; ee < 4; ++ee) {
        const int e = 4 * wave + ee;
        f32x4 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float s = red[(e * 4 + j) * 64 + lane];
#pragma unroll
            for (int w = 1; w < 4; ++w) s += red[w * RED + (e * 4 + j) * 64 + lane];
            v[j] = s;
        }
        const int row = 8 * wave + 4 * h + ee;
        if (row >= g.M || col >= g.N) continue;
        if (g.split_k > 1) *reinterpret_cast<f32x4 *>(g.ws + (((int64_t)slice * g.batch + batch) * g.M + row) * g.N + col) = v;
        else finish(v, row, col);
    }
    if (g.split_k == 1) return;

    // ---- several K slices: count in; whoever completes the count adds the slices up ----------------------------------
    // All slices of this unit run on this XCD: a partial tile is visible to them once its stores have been
    // acknowledged by the L2, and is read from there (sc1: past the reader's L1).  The counter lives in the L2 too.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) arrived_before = atomicInc(g.sk_flags + unit, (unsigned)g.split_k - 1);  // wraps to 0 with the last
    __syncthreads();
    if (arrived_before != (unsigned)g.split_k - 1) return;
    const int slice_bytes = g.batch * g.M * g.N * 4;  // (the whole workspace is below 2 GB: checked at launch)
    const __amdgpu_buffer_rsrc_t ws = __builtin_amdgcn_make_buffer_rsrc(g.ws, 0, -1, 0x00020000);
    constexpr int PIECES = FR_ROWS * FR_COLS / 4 / 256;
    f32x4 sum[PIECES];
    int off[PIECES];
#pragma unroll
    for (int p = 0; p < PIECES; ++p) {
        const int idx = tid + 256 * p;
        const int row = min(idx >> 5, g.M - 1), c = min(n0 + 4 * (idx & 31), g.N - 4);  // (clamped ones are not stored)
        off[p] = ((batch * g.M + row) * g.N + c) * 4;
        sum[p] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
    // four slices at a time, every load of them in flight together; slices beyond the last repeat it and add nothing
    for (int s0 = 0; s0 < g.split_k; s0 += 4) {
        f32x4 x[4][PIECES];
#pragma unroll
        for (int ds = 0; ds < 4; ++ds)
#pragma unroll
            for (int p = 0; p < PIECES; ++p) x[ds][p] = fr_load_l2(ws, off[p] + min(s0 + ds, g.split_k - 1) * slice_bytes);
#pragma unroll
        for (int ds = 0; ds < 4; ++ds)
#pragma unroll
            for (int p = 0; p < PIECES; ++p)
                if (s0 + ds < g.split_k) sum[p] += x[ds][p];
    }
#pragma unroll
    for (int p = 0; p < PIECES; ++p) {
        const int idx = tid + 256 * p;
        const int row = idx >> 5, c = n0 + 4 * (idx & 31);
        if (row < g.M && c < g.N) finish(sum[p], row, c);
    }
}

static bool fr_aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// 9 to 32 rows of a K-contiguous A against an N-contiguous W, everything in whole 16-byte pieces.
bool gemm_fewrows_eligible(const GemmLaunch &g, int amode, int bmode) {
    if (amode != 0 || bmode != 1 || g.M <= 8 || g.M > FR_ROWS || g.epilogue > MNI_EPI_BIAS_GELU) return false;
    if (g.K < 64 || g.K % 8 != 0 || g.N < FR_COLS || g.N % 4 != 0) return false;
    if (g.a_rs % 4 != 0 || g.b_rs % 4 != 0 || g.a_bs % 4 != 0 || g.b_bs % 4 != 0) return false;
    if (!fr_aligned16(g.A) || !fr_aligned16(g.B)) return false;
    if (g.ldc % 4 != 0 || g.c_bs % 4 != 0 || !fr_aligned16(g.C)) return false;
    if (g.epilogue != MNI_EPI_NONE && !fr_aligned16(g.bias)) return false;
    return true;
}

// g.tiles_n = column groups of 128; g.split_k slices of g.k_per_slice (a multiple of 32).
int launch_gemm_fewrows(const GemmLaunch &g, int amode, int bmode) {
    if (!gemm_fewrows_eligible(g, amode, bmode))
        return set_error(MNI_ERR_INVALID, "sgemm: the few-rows kernel takes 9 to 32 rows of a K-contiguous A against an N-contiguous B, "
                                          "K %% 8 == 0, N %% 4 == 0, 16-byte aligned");
    if (g.tiles_n != (g.N + FR_COLS - 1) / FR_COLS || g.split_k < 1 || g.k_per_slice % 32 != 0 || g.k_per_slice <= 0 ||
        (int64_t)g.split_k * g.k_per_slice < g.K || (g.split_k > 1 && (!g.ws || !g.sk_flags)) ||
        (int64_t)g.split_k * g.batch * g.M * g.N * 4 >= 0x7fffffffLL)
        return set_error(MNI_ERR_INVALID, "sgemm: few-rows kernel launched with a wrong plan");
    const int64_t units = (int64_t)g.tiles_n * g.batch;
    const int64_t blocks = 8 * ((units + 7) / 8) * g.split_k;  // every XCD gets the same number of units, the last ones empty
    if (blocks <= 0) return MNI_OK;
    if (blocks > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "sgemm: too many workgroups (%lld)", (long long)blocks);
    MNI_KERNEL_LAUNCH(gemm_fewrows_kernel, dim3((unsigned)blocks), dim3(256), 0, ctx().stream, g);
    return check_launch("gemm_fewrows_kernel");
}

}  // namespace mni
