// Dense fp32 GEMM for gfx950 on the MFMA matrix cores.
//
//   C[b] = epilogue( op(A)[b] (M x K)  *  op(B)[b] (K x N) )
//
// Replaces cuBLAS gemm / gemm_strided_batched of the reference's cuda arm
// (src/native/src/ops/matmul.rs:150-189) together with the permute_f32
// transposes that feed its backward products (:287-326).
//
// Tiling.  A workgroup of 256 threads (4 wavefronts, 2 x 2) owns a 128 x 128
// tile of C and walks K in steps of 32.  Each wavefront owns 64 x 64 as 2 x 2
// blocks of v_mfma_f32_32x32x2_f32 (16 accumulator VGPRs per block).  Narrow
// or short-K products use 64-wide tile sides (one MFMA block per wavefront along
// that side) from the same template.  Tiles are
// staged through LDS, double-buffered, one barrier per K step.  Global loads
// run a full K step ahead: the registers that carried tile t+1 into LDS during
// the last MFMAs of step t are refilled with tile t+2 right away, so a load has
// a whole step of MFMAs to land before it is needed.
//
// LDS layout and operand layouts (transposes folded into the load path).  The
// MFMA takes k = lane/32 from each lane, so a lane feeds four consecutive MFMAs
// from four K values of one row (m for A, n for B); lane half h contracts
// k = 8c+4h+j at MFMA j of chunk c for both operands, and the order of the K
// sum is the only thing that differs from a textbook loop.
// An operand whose K axis has unit stride (A row-major, or B given as its
// transpose) is loaded with 16-byte loads along K and stored "K-quad major",
//     tile[k/4][row][k%4]        (one float4 per row),
// so that one ds_read_b128 gives a lane its four K values and the 32 lanes of a
// half-wave read 32 consecutive float4 (conflict-free).
// An operand whose M/N axis has unit stride (B row-major, or A given as its
// transpose) is loaded with 16-byte loads along M/N and stored as it comes,
//     tile[k][row],
// and a lane gathers its four K values with four 4-byte reads (32 consecutive
// floats per half-wave, the halves 32 banks apart).  Nothing is transposed in
// registers: LDS instructions are free where vector-ALU instructions are not
// (see the K loop below).
// The 16-byte loads need no more than the 4-byte alignment every float has (the
// memory system splits a load that straddles a cache line), so odd leading
// dimensions and offset bases take these paths too.  Anything else (neither
// axis contiguous, K tails, edges of an M/N-contiguous operand off a multiple
// of 4) takes guarded scalar loads into the same register layout.
//
// K loop.  Tile kt+1 sits in staging registers while tile kt is multiplied out
// of LDS; in the last quarter of a step the staged tile goes to the other LDS
// stage and tile kt+2 is requested, so a request has a whole step to arrive
// (the steady form deals these transfers out in pieces, one or two behind each
// MFMA of that quarter; LDS is read in the first three quarters and written
// in the last).
// The loop exists twice.  The general form chooses between fast and guarded
// loads per step.  The steady form (whole K steps; a partial last step and the
// two before it are left to the general form) has no such choice and loads
// unconditionally: when the staging registers have two possible producers the
// compiler merges them with register copies that wait for the data right
// behind the request, which stalls every step for a memory round trip.  The
// steady form is also free of vector-ALU instructions: on this chip every one
// of them is paid for in fp32 MFMA issue time (measured: one v_mov per MFMA
// takes 8 % off a loop of MFMAs, an address add 15 %; LDS accesses, buffer
// loads and scalar instructions take nothing).  So it is unrolled over the two
// LDS stages (every LDS address a fixed register plus an immediate), loads go
// through buffer instructions whose moving parts (tile base, K advance, row
// pitch) are scalar, and nothing is shuffled between load and LDS store.
//
// Work distribution.  Classic form: one workgroup per (tile, batch, K slice);
// with more than one slice the partials go to a workspace and a second kernel
// adds them.  Stream-K form (Osama et al., "Stream-K", PPoPP'23, restricted to
// one XCD at a time): a fixed grid of resident workgroups; every XCD owns a
// contiguous run of whole tiles.  Whole rounds of one tile per workgroup are
// done tile by tile; the tiles that do not fill a round (with one full round,
// when there is one) have their K steps dealt evenly over the XCD's
// workgroups, so a workgroup's share may start and end in the middle of a tile.
// A workgroup walks its share backwards: the piece at the end (the head of a
// tile somebody else finishes) is computed first and parked in the workspace
// with an arrival mark; whole tiles follow; the piece at the start (the tail
// of a tile begun by lower-numbered workgroups) comes last, by which time
// their partials arrived long ago.  Whoever holds a tile's last K step adds
// the parked partials in workgroup order and runs the epilogue, so the sum
// order is fixed by the shape alone.  Partials never leave the XCD's L2, and
// a workgroup only ever waits for lower-numbered (earlier dispatched) ones.
#include "common.h"
#include "gemm_internal.h"
#include <type_traits>

namespace mni {

typedef float floatx16 __attribute__((ext_vector_type(16)));

static constexpr int BK = 32;
static constexpr int KQ = BK / 4;           // K quads per tile
static constexpr int PAD = 2;               // float4 of padding per K-quad slice
static constexpr int NTHREADS = 256;
static constexpr int SK_WAIT_LIMIT = 1 << 20;  // polls before a finisher gives up, writes NaN and sets the status word

__device__ __forceinline__ unsigned load_mark(const unsigned *p) {
    // sc1: answered by the XCD's L2, never by this CU's L1
    unsigned v;
    asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}

// Row r of a tile sits at float4 slot r ^ ((r >> 4) & 3) of its K-quad slice.
// Within an aligned group of 16 rows this is a permutation, so the MFMA operand
// reads (16 consecutive rows per LDS pass) stay conflict-free; it spreads the
// 16 rows 4*j + i that the micro-tile stores write in one pass over all 16
// bank groups (they would otherwise collide four ways).
__device__ __forceinline__ int lds_row(int r) { return r ^ ((r >> 4) & 3); }

// ---- global -> register loads ---------------------------------------------
// A tile side has ROWS = 256, 128 or 64 rows (m for A, n for B) and BK = 32 K
// values: ROWS / 32 16-byte pieces per thread.
// Register layout LAYOUT 0 (K contiguous): thread owns float4 #(tid + 256 i),
//   i < ROWS/32, where float4 #f is row f/8, K quad f%8: four K values of one
//   row, which is what one LDS slot holds.
// Register layout LAYOUT 1 (M/N contiguous): thread owns rows 4 r4 .. 4 r4 + 3,
//   r4 = tid % (ROWS/4), at the K values tid / (ROWS/4) + (1024 / ROWS) i,
//   i < ROWS/32: one 16-byte load along M/N each.  Its four components belong
//   to four different LDS slots and are stored there one by one (4-byte LDS
//   stores).  Nothing is shuffled in registers in either layout: every
//   vector-ALU instruction in the K loop takes its cycles from the fp32 MFMAs (a
//   v_mov per MFMA costs 8 % of the matrix rate on this chip; loads, LDS
//   traffic and scalar work cost nothing), so the loop is built to contain none.
template <int ROWS> __device__ constexpr int stage_regs() { return ROWS / 32 > 4 ? ROWS / 32 : 4; }
template <int ROWS> __device__ constexpr int k_stride() { return 4 * NTHREADS / ROWS; }  // K rows covered per pass (layout 1)

// Rows at or beyond `rows` (an edge tile; a multiple of 4 for layout 1) are
// read from the last valid row or row quad instead: what they contribute lands
// in accumulator rows / columns that the epilogue never stores.
template <int LAYOUT, int ROWS>
__device__ __forceinline__ void load_fast(const float *__restrict__ p, int64_t ld, int rows, int tid, float4 (&v)[stage_regs<ROWS>()]) {
#pragma unroll
    for (int i = 0; i < ROWS / 32; ++i) {
        if (LAYOUT == 0) {
            int f = tid + NTHREADS * i;
            int row = min(f >> 3, rows - 1), q = f & 7;
            v[i] = *reinterpret_cast<const float4 *>(p + (int64_t)row * ld + 4 * q);
        } else {
            constexpr int R4 = ROWS / 4;
            const int r4 = min(tid % R4, rows / 4 - 1), k = tid / R4 + k_stride<ROWS>() * i;
            v[i] = *reinterpret_cast<const float4 *>(p + 4 * r4 + (int64_t)k * ld);
        }
    }
}

// Guarded element-wise load: element (row, k) lives at p[row * rs + k * cs];
// rows >= rmax or k >= kmax read as zero.
template <int LAYOUT, int ROWS>
__device__ __forceinline__ void load_guarded(const float *__restrict__ p, int64_t rs, int64_t cs, int rmax,
                                             int kmax, int tid, float4 (&v)[stage_regs<ROWS>()]) {
    // Edge tiles and K tails only.  The empty asm makes the element addresses
    // get computed here, on use: computed once ahead of the K loop they would
    // occupy sixteen register pairs for the whole loop.
    asm volatile("" : "+v"(tid));
#pragma unroll
    for (int i = 0; i < ROWS / 32; ++i) {
        float t[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            int row, k;
            if (LAYOUT == 0) {
                const int f = tid + NTHREADS * i;
                row = f >> 3, k = 4 * (f & 7) + e;
            } else {
                row = 4 * (tid % (ROWS / 4)) + e, k = tid / (ROWS / 4) + k_stride<ROWS>() * i;
            }
            t[e] = (row < rmax && k < kmax) ? p[(int64_t)row * rs + (int64_t)k * cs] : 0.0f;
        }
        v[i] = make_float4(t[0], t[1], t[2], t[3]);
    }
}

// ---- register -> LDS, LDS -> MFMA operands -----------------------------------
// A tile stage in LDS, by layout:
//   0: float4 tile[K quad][row] (pitch ROWS + PAD slots): a register quad is one
//      slot, and one ds_read_b128 gives a lane the K values of four MFMAs;
//   1: float  tile[k][row] (pitch ROWS + 8 floats): a register quad (four rows
//      at one K value) is 16 contiguous bytes, and a lane gathers its four K
//      values with four 4-byte reads.  The pitch puts the rows of K value k + 4
//      -- what the other half of the wavefront reads -- 32 banks further on.
// LDS instructions cost the matrix pipe nothing; a transpose in registers
// would.
template <int LAYOUT, int ROWS>
__device__ constexpr int stage_slots() { return LAYOUT == 0 ? KQ * (ROWS + PAD) : BK * (ROWS + 8) / 4; }  // float4 per stage

template <int LAYOUT, int ROWS>
__device__ __forceinline__ void store_piece(float4 *__restrict__ tile, int tid, int i, const float4 &v) {
    if (LAYOUT == 0) {
        const int f = tid + NTHREADS * i;
        tile[(f & 7) * (ROWS + PAD) + lds_row(f >> 3)] = v;
    } else {
        const int k = tid / (ROWS / 4) + k_stride<ROWS>() * i;
        tile[k * ((ROWS + 8) / 4) + tid % (ROWS / 4)] = v;
    }
}

template <int LAYOUT, int ROWS>
__device__ __forceinline__ void store_lds(float4 *__restrict__ tile, int tid, const float4 (&v)[stage_regs<ROWS>()]) {
#pragma unroll
    for (int i = 0; i < ROWS / 32; ++i) store_piece<LAYOUT, ROWS>(tile, tid, i, v[i]);
}

// What a lane keeps per MFMA block row: where row `row` of the tile sits in a stage.
template <int LAYOUT>
__device__ __forceinline__ int frag_row(int row) { return LAYOUT == 0 ? lds_row(row) : row; }

// K values 8 c + 4 h + 0..3 of the row: the operands of the four MFMA groups of chunk c for lane half h.
template <int LAYOUT, int ROWS>
__device__ __forceinline__ float4 frag_load(const float4 *__restrict__ tile, int c, int h, int frow) {
    if (LAYOUT == 0) return tile[(2 * c + h) * (ROWS + PAD) + frow];
    const float *t = reinterpret_cast<const float *>(tile) + (8 * c + 4 * h) * (ROWS + 8) + frow;
    return make_float4(t[0], t[ROWS + 8], t[2 * (ROWS + 8)], t[3 * (ROWS + 8)]);
}

// ---- the steady K loop's transfers -------------------------------------------
// In the steady loop a tile side moves in pieces dealt out behind the MFMAs:
// first the ROWS/32 LDS stores of the staged tile, then the loads that refill
// the staging registers.  The loads are buffer loads: the tile's base address
// and the K advance sit in the scalar resource descriptor, offsets that depend
// on the leading dimension in a scalar offset, and the only vector register
// involved is a per-thread byte offset computed once ahead of the loop.
typedef float floatx4 __attribute__((ext_vector_type(4)));

struct StageAddr {
    int voff[8];  // layout 0: byte offset of piece i; layout 1: voff[0] = byte offset of the thread's row quad at its first K row
    int ldb;      // leading dimension in bytes
};

template <int LAYOUT, int ROWS>
__device__ __forceinline__ StageAddr stage_addr(int64_t ld, int rows, int tid) {
    StageAddr s;
    s.ldb = (int)ld * 4;
    if (LAYOUT == 0) {
#pragma unroll
        for (int i = 0; i < ROWS / 32; ++i) {
            const int f = tid + NTHREADS * i;
            s.voff[i] = (min(f >> 3, rows - 1) * (int)ld + 4 * (f & 7)) * 4;
        }
    } else {
        s.voff[0] = 16 * min(tid % (ROWS / 4), rows / 4 - 1) + (tid / (ROWS / 4)) * s.ldb;
    }
    return s;
}

// Whether the offsets above fit the 32-bit offset fields of a buffer load.
template <int ROWS>
__device__ __forceinline__ bool stage_addr_fits(int64_t ld) { return ld > 0 && ld * 4 * (ROWS > BK ? ROWS : BK) < (int64_t)0x7fffffff; }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t stage_rsrc(const float *p) {
    // raw buffer: stride 0, no range limit (rows are clamped by the caller), 32-bit data format
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p), 0, -1, 0x00020000);
}

template <int ROWS>
__device__ constexpr int tile_pieces() { return 2 * (ROWS / 32); }

template <int LAYOUT, int ROWS>
__device__ __forceinline__ void tile_piece(int x, float4 *__restrict__ tile, __amdgpu_buffer_rsrc_t rsrc, const StageAddr &sa,
                                           int tid, float4 (&v)[stage_regs<ROWS>()]) {
    constexpr int NV = ROWS / 32;
    if (x < NV) {
        store_piece<LAYOUT, ROWS>(tile, tid, x, v[x]);
    } else {
        const int i = x - NV;
        const floatx4 t = __builtin_bit_cast(floatx4, LAYOUT == 0 ? __builtin_amdgcn_raw_buffer_load_b128(rsrc, sa.voff[i], 0, 0)
                                                                  : __builtin_amdgcn_raw_buffer_load_b128(rsrc, sa.voff[0], k_stride<ROWS>() * i * sa.ldb, 0));
        v[i] = make_float4(t.x, t.y, t.z, t.w);
    }
}

// GELU (tanh approximation, src/native/src/ops/activation.rs:15-28) in the epilogues.  With u = s (x + c x^3),
// s = sqrt(2/pi), c = 0.044715:  0.5 (1 + tanh u) = 1 / (1 + e^{-2u}) =: sig, so
//     gelu(x)  = x sig
//     gelu'(x) = sig + 0.5 x sech^2(u) u' = sig (1 + x (1 - sig) 2u'),   2u' = 2s + 6sc x^2,
// through the hardware's exp2 and reciprocal (exact limits at both ends, absolute error ~1e-6): seven instructions for
// the value, eleven for the derivative.  The count matters: an epilogue's vector-ALU instructions are paid for in MFMA
// time of the workgroup that shares the SIMDs (the library's tanhf, some forty instructions, made the fused GELU
// products 25 us slower than the plain ones plus a separate pass).
__device__ __forceinline__ float gelu_sig(float x, float x2) {
    const float c0 = -2.0f * 0.7978845608028654f * 1.4426950408889634f;             // -2 s log2(e)
    const float c1 = -2.0f * 0.7978845608028654f * 0.044715f * 1.4426950408889634f;  // -2 s c log2(e)
    const float e = __builtin_amdgcn_exp2f(x * __builtin_fmaf(x2, c1, c0));           // e^{-2u}
    return __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ float gelu_tanh(float x) { return x * gelu_sig(x, x * x); }

__device__ __forceinline__ float gelu_tanh_grad(float x) {
    const float x2 = x * x;
    const float sig = gelu_sig(x, x2);
    const float du2 = __builtin_fmaf(x2, 6.0f * 0.7978845608028654f * 0.044715f, 2.0f * 0.7978845608028654f);  // 2u'
    return sig * __builtin_fmaf(x * du2, 1.0f - sig, 1.0f);
}

__device__ __forceinline__ float pick(const float4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }

// MODE: 0 = K axis contiguous, 1 = M/N axis contiguous, 2 = arbitrary strides
// (always guarded scalar loads, layout 0).
// TM x TN: 32 x 32 MFMA blocks per wavefront; the workgroup tile is
// (64 TM) x (64 TN): 128 x 128 for the dense case, 64-wide sides for narrow or
// short-K products where smaller tiles waste less and fill the machine better.
// SK: the stream-K form (a loop over this workgroup's segments); otherwise the
// body runs once for the (tile, batch, slice) named by the workgroup id.
typedef const GemmLaunch __attribute__((address_space(4))) *LaunchPtr;

// float4 slots of LDS a workgroup needs: two stages of the A tile, two of the B tile; the epilogue reuses the
// block to turn the MFMA accumulator layout into row-contiguous 16-byte stores.
template <int AMODE, int BMODE, int TM, int TN>
__device__ constexpr int gemm_lds_slots() {
    return 2 * stage_slots<AMODE == 1 ? 1 : 0, 64 * TM>() + 2 * stage_slots<BMODE == 1 ? 1 : 0, 64 * TN>();
}

// The work of one workgroup.  gp: the launch descriptor in the kernel-argument segment (read through scalar
// loads, afresh for every stream-K segment, instead of being held in scalar registers across the K loop);
// wg / nwg: this workgroup's number and the number of workgroups of this product, numbered the way the
// hardware deals workgroups to XCDs (wg % 8 is the XCD); lds: gemm_lds_slots() float4.
// FRESH: the body runs inside a loop of its caller (as it does inside its own loop over stream-K segments): what a thread
// derives from its id is then derived afresh on every call instead of staying live across the K loop.
template <int AMODE, int BMODE, int TM, int TN, bool SK, bool FRESH = SK>
__device__ __forceinline__ void gemm_mfma_body(LaunchPtr gp, const unsigned wg, const unsigned nwg, float4 *__restrict__ lds) {
#define g (*gp)
    constexpr int AL = AMODE == 1 ? 1 : 0;
    constexpr int BL = BMODE == 1 ? 1 : 0;
    constexpr int BM = 64 * TM, BN = 64 * TN;
    constexpr int STAGE_A = stage_slots<AL, BM>(), STAGE_B = stage_slots<BL, BN>();
    auto stage_a = [&](int st) -> float4 * { return lds + st * STAGE_A; };
    auto stage_b = [&](int st) -> float4 * { return lds + 2 * STAGE_A + st * STAGE_B; };

    // ---- segments of work ----------------------------------------------------
    enum { ROLE_FULL = 0, ROLE_SLICE = 1, ROLE_PART = 2, ROLE_FINISH = 3 };
    const int tiles = g.tiles_m * g.tiles_n;
    const int ksteps = (g.K + BK - 1) / BK;
    // Stream-K.  The XCD's run of tiles splits into a stream-K region (its
    // first sk_tiles tiles, whose K steps are dealt evenly: this workgroup's
    // share is [seg_lo, seg_hi)) and whole rounds of one tile per workgroup
    // after it.  The region is what does not fill a round, plus one full
    // round when there is one, so that a share is at least a tile's worth.
    // Only seg_hi (end of what is left of the share) and dp_tile (next whole
    // tile) are carried from segment to segment; everything else is derived
    // again from the workgroup id at the top of a segment, which keeps the
    // scalar registers free across the K loop.
    int seg_hi = 0, dp_tile = 0;
    struct Share { int x, i, tile0, tiles, units, lo, hi, dp0; };
    auto share_of = [&](unsigned bid) {
        Share sh;
        sh.x = (int)(bid % g.sk_xcds);
        sh.i = (int)(bid / g.sk_xcds);
        const int total = tiles * g.batch;
        const int q = total / g.sk_xcds, rem = total % g.sk_xcds;
        sh.tile0 = sh.x < rem ? sh.x * (q + 1) : rem * (q + 1) + (sh.x - rem) * q;
        sh.tiles = q + (sh.x < rem ? 1 : 0);
        const int rounds = sh.tiles / g.sk_wpx, left = sh.tiles - rounds * g.sk_wpx;
        const int sk_tiles = left == 0 ? 0 : (rounds > 0 ? left + g.sk_wpx : left);
        sh.units = sk_tiles * ksteps;
        sh.lo = (int)((int64_t)sh.i * sh.units / g.sk_wpx);
        sh.hi = (int)((int64_t)(sh.i + 1) * sh.units / g.sk_wpx);
        sh.dp0 = sk_tiles + sh.i;
        return sh;
    };
    if (SK) {
        const Share sh = share_of(wg);
        seg_hi = sh.hi;
        dp_tile = sh.dp0;
        if (seg_hi <= sh.lo && dp_tile >= sh.tiles) return;
    }

    do {
    // Everything a thread derives from its id is derived again for every
    // segment (the empty asm hides that it never changes): hoisted out of the
    // segment loop, those addresses would stay live across it and spill.
    int tid = threadIdx.x;
    unsigned bid = wg;
    if (SK || FRESH) {
        asm volatile("" : "+v"(tid));
        asm volatile("" : "+s"(gp));
        asm volatile("" : "+s"(bid));
    }
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int r = lane & 31, h = lane >> 5;
    // float4 slots of this lane's A row blocks and B column blocks
    int a_row[TM], b_row[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i) a_row[i] = frag_row<AL>(wm * (32 * TM) + 32 * i + r);
#pragma unroll
    for (int j = 0; j < TN; ++j) b_row[j] = frag_row<BL>(wn * (32 * TN) + 32 * j + r);

    int64_t pid;
    int role, k_begin, k_end, slice = 0;
    // ROLE_FINISH: fin = c_first | c_count << 15, the workgroups (index within
    // the XCD) whose partials belong to this tile; bit 30 of fin: more segments follow
    int fin = 0;
    if (!SK) {
        // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.
        // Renumber so that every XCD works on one contiguous run of tiles.
        pid = wg;
        const int64_t total = nwg;
        const int64_t q = total >> 3, rr = total & 7;
        const int64_t x = pid & 7, i = pid >> 3;
        pid = (x < rr ? x * (q + 1) : rr * (q + 1) + (x - rr) * q) + i;
        role = g.split_k > 1 ? ROLE_SLICE : ROLE_FULL;
        k_begin = 0;  // set below from the slice
        k_end = 0;
    } else {
        const Share sh = share_of(bid);
        if (seg_hi > sh.lo) {
            const int lt = (seg_hi - 1) / ksteps;
            const int tstart = lt * ksteps;
            const int sb = sh.lo > tstart ? sh.lo : tstart;
            const int kb = sb - tstart, ke = seg_hi - tstart;
            pid = sh.tile0 + lt;
            role = ke < ksteps ? ROLE_PART : (kb == 0 ? ROLE_FULL : ROLE_FINISH);
            if (role == ROLE_FINISH) {
                const int c_first = (int)((((int64_t)tstart + 1) * g.sk_wpx - 1) / sh.units);  // owner of the tile's first K step
                fin = c_first | (sh.i - c_first) << 15;
            }
            k_begin = kb * BK;
            k_end = min(g.K, ke * BK);
            seg_hi = sb;
        } else {
            pid = sh.tile0 + dp_tile;
            dp_tile += g.sk_wpx;
            role = ROLE_FULL;
            k_begin = 0;
            k_end = g.K;
        }
        if (seg_hi > sh.lo || dp_tile < sh.tiles) fin |= 1 << 30;
    }
    // Tiles are walked in column-grouped order so that concurrently resident
    // tiles share A row panels and B column panels in the XCD's L2.
    const int z = (int)(pid / tiles);
    int t = (int)(pid - (int64_t)z * tiles);
    int batch = z;
    if (!SK) {
        batch = z / g.split_k;
        slice = z - batch * g.split_k;
        k_begin = slice * g.k_per_slice;
        k_end = min(g.K, k_begin + g.k_per_slice);
    }
    int tm, tn;
    {
        const int GROUP = 8;
        const int per_group = GROUP * g.tiles_n;
        const int gid = t / per_group;
        const int first = gid * GROUP;
        const int gsz = min(g.tiles_m - first, GROUP);
        const int in_group = t - gid * per_group;
        tm = first + in_group % gsz;
        tn = in_group / gsz;
    }
    const int m0 = tm * BM, n0 = tn * BN;
    const int klen = max(k_end - k_begin, 0);
    const int nkt = (klen + BK - 1) / BK;

    const float *__restrict__ Ap =
        g.A + (int64_t)(batch % g.a_bcount) * g.a_bs + (int64_t)m0 * g.a_rs + (int64_t)k_begin * g.a_cs;
    const float *__restrict__ Bp =
        g.B + (int64_t)(batch % g.b_bcount) * g.b_bs + (int64_t)n0 * g.b_cs + (int64_t)k_begin * g.b_rs;
    const int mrem = g.M - m0, nrem = g.N - n0;
    // Fast loads also serve an edge tile (rows beyond the edge re-read the last
    // valid ones), except that 16-byte loads along M/N need the edge on a
    // multiple of 4.
    const int a_rows = min(mrem, BM), b_rows = min(nrem, BN);
    const bool a_fast = AMODE == 0 || (AMODE == 1 && a_rows % 4 == 0);
    const bool b_fast = BMODE == 0 || (BMODE == 1 && b_rows % 4 == 0);
    // leading dimension seen by the fast loaders
    const int64_t a_ld = AMODE == 0 ? g.a_rs : g.a_cs;
    const int64_t b_ld = BMODE == 0 ? g.b_cs : g.b_rs;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    float4 ra[stage_regs<BM>()], rb[stage_regs<BN>()];

    auto load_a = [&](int kt) {  // A tile: rows = m, element (m, k) at Ap[m * a_rs + k * a_cs]
        const int k0 = kt * BK;
        const int krem = klen - k0;
        if (a_fast && krem >= BK) {
            if (AMODE == 0) load_fast<0, BM>(Ap + (int64_t)k0, a_ld, a_rows, tid, ra);
            else load_fast<1, BM>(Ap + (int64_t)k0 * a_ld, a_ld, a_rows, tid, ra);
        } else {
            load_guarded<AL, BM>(Ap + (int64_t)k0 * g.a_cs, g.a_rs, g.a_cs, mrem, krem, tid, ra);
        }
    };
    auto load_b = [&](int kt) {  // B tile: rows = n, element (n, k) at Bp[n * b_cs + k * b_rs]
        const int k0 = kt * BK;
        const int krem = klen - k0;
        if (b_fast && krem >= BK) {
            if (BMODE == 0) load_fast<0, BN>(Bp + (int64_t)k0, b_ld, b_rows, tid, rb);
            else load_fast<1, BN>(Bp + (int64_t)k0 * b_ld, b_ld, b_rows, tid, rb);
        } else {
            load_guarded<BL, BN>(Bp + (int64_t)k0 * g.b_rs, g.b_cs, g.b_rs, nrem, krem, tid, rb);
        }
    };

    // Prologue: tile 0 goes to LDS stage 0, tile 1 into the staging registers.
    if (nkt > 0) {
        load_a(0);
        load_b(0);
        store_lds<AL, BM>(stage_a(0), tid, ra);
        store_lds<BL, BN>(stage_b(0), tid, rb);
        if (nkt > 1) { load_a(1); load_b(1); }
    }
    __syncthreads();

    constexpr int NCHUNK = KQ / 2;  // chunks of 8 K values

    // One chunk = 8 K values = 4 groups of TM x TN MFMAs (group j uses element
    // j of each operand float4).  The ds_read_b128 of the NEXT chunk are issued
    // after the first three groups, and in the last chunk of a step the LDS
    // writes of the next stage take their place, so LDS traffic is spread under
    // the MFMAs instead of bunching up in front of a wait.  sched_barrier keeps
    // the compiler from regrouping them.
    float4 fa[TM], fb[TN];  // fragments in use
    float4 na[TM], nb[TN];  // fragments of the next chunk
    // Both resident wavefronts of a SIMD issue at the default priority: raising
    // it around the MFMAs paid off only while the K loop still stalled on its
    // loads, and costs 2 % at 4096^3 now that it does not.
    auto mfma_group = [&](int j) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int jj = 0; jj < TN; ++jj)
                acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(pick(fa[i], j), pick(fb[jj], j), acc[i][jj], 0, 0, 0);
    };
    // The first three quarters of a K step: MFMAs of chunk c with the fragment
    // reads of chunk c + 1 between the groups.
    auto chunk = [&](const float4 *As, const float4 *Bs, int c) {
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TM; ++i) na[i] = frag_load<AL, BM>(As, c + 1, h, a_row[i]);
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(1);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < (TN + 1) / 2; ++j) nb[j] = frag_load<BL, BN>(Bs, c + 1, h, b_row[j]);
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(2);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = (TN + 1) / 2; j < TN; ++j) nb[j] = frag_load<BL, BN>(Bs, c + 1, h, b_row[j]);
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(3);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = na[i];
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j] = nb[j];
    };

    // Steady form of a K step (every load a fast one; the stage is a
    // compile-time constant, the loop below is unrolled over both, so that
    // every LDS address is a register fixed ahead of the loop plus an immediate).
    // The staged tile goes to LDS and tile kt + 2 is requested piece by piece,
    // one or two pieces behind each MFMA of the last chunk, so that none of it
    // has to be issued with the matrix pipe idle.  The last two steps park and
    // fetch the final tile again, which nobody reads: the staging registers have
    // one producer, and no branch on which the compiler could merge two with
    // register copies that wait for the data right behind the request.
    const StageAddr sa_a = stage_addr<AL, BM>(a_ld, a_rows, tid), sa_b = stage_addr<BL, BN>(b_ld, b_rows, tid);
    auto steady_step = [&](auto stage, int kt) {
        constexpr int cur = decltype(stage)::value;
        const int kt2 = min(kt + 2, nkt - 1);
        const float4 *As = stage_a(cur), *Bs = stage_b(cur);
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = frag_load<AL, BM>(As, 0, h, a_row[i]);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j] = frag_load<BL, BN>(Bs, 0, h, b_row[j]);
#pragma unroll
        for (int c = 0; c < NCHUNK - 1; ++c) chunk(As, Bs, c);
        constexpr int PA = tile_pieces<BM>(), PB = tile_pieces<BN>();
        constexpr int SLOTS = 4 * TM * TN, PER = (PA + PB + SLOTS - 1) / SLOTS;
        const __amdgpu_buffer_rsrc_t ra_src = stage_rsrc(AMODE == 0 ? Ap + (int64_t)kt2 * BK : Ap + (int64_t)kt2 * BK * a_ld);
        const __amdgpu_buffer_rsrc_t rb_src = stage_rsrc(BMODE == 0 ? Bp + (int64_t)kt2 * BK : Bp + (int64_t)kt2 * BK * b_ld);
        int slot = 0;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int jj = 0; jj < TN; ++jj) {
                    __builtin_amdgcn_sched_barrier(0);
                    acc[i][jj] = __builtin_amdgcn_mfma_f32_32x32x2f32(pick(fa[i], j), pick(fb[jj], j), acc[i][jj], 0, 0, 0);
                    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                    for (int x = slot * PER; x < (slot + 1) * PER; ++x) {
                        if (x < PA) tile_piece<AL, BM>(x, stage_a(cur ^ 1), ra_src, sa_a, tid, ra);
                        else if (x < PA + PB) tile_piece<BL, BN>(x - PA, stage_b(cur ^ 1), rb_src, sa_b, tid, rb);
                    }
                    ++slot;
                }
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    };

    // General form: chooses between fast and guarded loads per step.
    auto general_step = [&](int kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < nkt, more2 = kt + 2 < nkt;
        const float4 *As = stage_a(cur), *Bs = stage_b(cur);
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[i] = frag_load<AL, BM>(As, 0, h, a_row[i]);
#pragma unroll
        for (int j = 0; j < TN; ++j) fb[j] = frag_load<BL, BN>(Bs, 0, h, b_row[j]);
#pragma unroll
        for (int c = 0; c < NCHUNK - 1; ++c) chunk(As, Bs, c);
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(0);
        __builtin_amdgcn_sched_barrier(0);
        if (more) {
            // The staging registers hold tile kt+1 (requested a whole K step
            // ago); once they are in LDS they are refilled with tile kt+2.
            store_lds<AL, BM>(stage_a(cur ^ 1), tid, ra);
            if (more2) load_a(kt + 2);
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(1);
        __builtin_amdgcn_sched_barrier(0);
        if (more) {
            store_lds<BL, BN>(stage_b(cur ^ 1), tid, rb);
            if (more2) load_b(kt + 2);
        }
        __builtin_amdgcn_sched_barrier(0);
        mfma_group(2);
        mfma_group(3);
        __builtin_amdgcn_sched_barrier(0);
        __syncthreads();
    };
    // A tile whose fast loads fit the buffer-load offsets runs pairs of steady
    // steps; when K ends in a partial step, up to the step that requests that
    // last tile (two steps ahead), and the general form takes what remains.
    int nsteady = 0;
    if (a_fast && b_fast && stage_addr_fits<BM>(a_ld) && stage_addr_fits<BN>(b_ld))
        nsteady = (klen % BK == 0 ? nkt : max(nkt - 3, 0)) & ~1;
    for (int kt = 0; kt < nsteady; kt += 2) {
        steady_step(std::integral_constant<int, 0>(), kt);
        steady_step(std::integral_constant<int, 1>(), kt + 1);
    }
    for (int kt = nsteady; kt < nkt; ++kt) general_step(kt);

    // ---- epilogue -----------------------------------------------------------
    // A 32 x 32 MFMA block leaves lane l with column l%32 and rows
    // 8*(e/4) + 4*(l/32) + e%4, e = 0..15.  Storing that directly costs one
    // 4-byte store per value; instead every wavefront passes its 32-row strips
    // through a private LDS patch and writes them back out as 16-byte stores
    // along the rows (4x fewer store instructions, which is what bounds
    // short-K, output-heavy products).
    float *__restrict__ Cb;
    int64_t ldc;
    const bool partial = role == ROLE_SLICE;
    if (partial) {
        Cb = g.ws + ((int64_t)slice * g.batch + batch) * (int64_t)g.M * g.N;
        ldc = g.N;
    } else {
        Cb = g.C + (int64_t)batch * g.c_bs;
        ldc = g.ldc;
    }
    constexpr int WN = 32 * TN;          // columns of a wavefront's strip
    constexpr int PW = WN + 4;           // patch row pitch in floats (16-byte multiple)
    constexpr int LANES_PER_ROW = WN / 4;
    constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
    float *patch = reinterpret_cast<float *>(lds) + wave * (32 * PW);
    const int prow = lane / LANES_PER_ROW, pc4 = lane % LANES_PER_ROW;
    const int coll = wn * WN + 4 * pc4;  // column within the tile
    const int col = n0 + coll;
    // 16-byte stores (and the loads of an accumulating epilogue) go to any
    // 4-byte aligned address, as the operand loads do
    constexpr bool vec_ok = true;
    float bias4[4] = {0.f, 0.f, 0.f, 0.f};
    if (!partial && !(SK && role == ROLE_PART) && g.epilogue != MNI_EPI_NONE) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (col + e < g.N) bias4[e] = g.bias[col + e];
    }
    // Stream-K: a finisher makes sure the partials of its tile have arrived
    // (they were parked at the very start of their owners' lives).
    bool lost = false;
    const int c_first = fin & 0x7fff, c_count = (fin >> 15) & 0x7fff;
    const int sk_x = SK ? (int)(bid % g.sk_xcds) : 0;
    if (SK && role == ROLE_FINISH) {
        bool ok = true;
        if (tid < c_count) {
            const unsigned *mark = g.sk_flags + (sk_x + g.sk_xcds * (c_first + tid));
            ok = false;
            for (int spin = 0; spin < SK_WAIT_LIMIT; ++spin) {
                if (load_mark(mark) == g.sk_epoch) { ok = true; break; }
                __builtin_amdgcn_s_sleep(4);
            }
        }
        lost = __syncthreads_or(!ok) != 0;
        // Tell the host: the next call that waits for the stream fails with this code.
        if (lost && tid == 0) *g.status = DEVICE_STATUS_STREAMK_WAIT;
    }
    float *const slot = g.ws + (int64_t)bid * (BM * BN);  // ROLE_PART: where this workgroup parks its tile
    // Fused backward of a GELU layer (MNI_EPI_DGELU, whole tiles only): the lane's four columns, summed
    // over the rows of this wavefront's strip, on the way to the bias gradient.
    const bool dual = !SK && !partial && g.epilogue == MNI_EPI_BIAS_GELU_DUAL;
    const bool dgelu = !SK && !partial && g.epilogue == MNI_EPI_DGELU;
    float csum[4] = {0.f, 0.f, 0.f, 0.f};
    // The saved pre-activations of this wavefront's part of the tile are requested here, all at once, so that the
    // strips below find them in registers instead of waiting for a memory round trip per strip (columns in whole
    // quads only: N % 4 == 0; rows and quads beyond the edge re-read the last valid ones and are not used).
    constexpr int PASSES = 32 / ROWS_PER_PASS;
    float4 zpre[TM][PASSES];
    const bool zvec = dgelu && g.N % 4 == 0 && g.N >= 4;
    if (zvec) {
        const float *zb = g.aux_in + (int64_t)batch * g.c_bs + min(col, g.N - 4);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int pass = 0; pass < PASSES; ++pass) {
                const int row = min(m0 + wm * (32 * TM) + 32 * i + prow + ROWS_PER_PASS * pass, g.M - 1);
                zpre[i][pass] = *reinterpret_cast<const float4 *>(zb + (int64_t)row * ldc);
            }
    }
    // All wavefronts are past their last LDS read (barrier at the end of the K loop), and a patch belongs to one
    // wavefront: its lanes exchange values through it, which needs the LDS accesses kept in program order (they are
    // executed in order per wavefront) but no workgroup barrier.
    auto wave_sync = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // One 32-row strip of the wavefront's blocks at a time.  The strip index is a compile-time constant (a
    // lambda called once per value, not a loop): were the loop left rolled -- the body is long, and with
    // four strips the unroller declines -- the accumulators would be indexed at run time, live in scratch
    // memory, and every MFMA of the K loop would be followed by a store of its result.
    auto epilogue_strip = [&](auto strip) {
        constexpr int i = decltype(strip)::value;
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) patch[(8 * (e >> 2) + 4 * h + (e & 3)) * PW + 32 * j + r] = acc[i][j][e];
        wave_sync();
#pragma unroll
        for (int pass = 0; pass < 32 / ROWS_PER_PASS; ++pass) {
            const int lr = prow + ROWS_PER_PASS * pass;
            const int rowl = wm * (32 * TM) + 32 * i + lr;  // row within the tile
            const int row = m0 + rowl;
            const float4 t4 = *reinterpret_cast<const float4 *>(patch + lr * PW + 4 * pc4);
            float v[4] = {t4.x, t4.y, t4.z, t4.w};
            if (SK && role == ROLE_PART) {
                *reinterpret_cast<float4 *>(slot + rowl * BN + coll) = t4;
                continue;
            }
            if (SK && role == ROLE_FINISH) {
                // four partials requested at a time, added in workgroup order
                for (int c0 = 0; c0 < c_count; c0 += 4) {
                    float4 pv[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const float *ps = g.ws + (int64_t)(sk_x + g.sk_xcds * (c_first + c0 + j)) * (BM * BN);
                        pv[j] = c0 + j < c_count ? *reinterpret_cast<const float4 *>(ps + rowl * BN + coll)
                                                 : make_float4(0.f, 0.f, 0.f, 0.f);
                    }
#pragma unroll
                    for (int j = 0; j < 4; ++j) { v[0] += pv[j].x; v[1] += pv[j].y; v[2] += pv[j].z; v[3] += pv[j].w; }
                }
                if (lost) v[0] = v[1] = v[2] = v[3] = __builtin_nanf("");
            }
            if (row < g.M && col < g.N) {
                float *dst = Cb + (int64_t)row * ldc + col;
                if (dual) {
                    // C keeps the product; the activated value goes to the second output, laid out like C
                    float *dst2 = g.aux_out + (int64_t)batch * g.c_bs + (int64_t)row * ldc + col;
                    float w[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) w[e] = gelu_tanh(v[e] + bias4[e]);
                    if (col + 3 < g.N) {
                        typedef float f32x4_t __attribute__((ext_vector_type(4)));
                        const f32x4_t o4 = {w[0], w[1], w[2], w[3]};
                        __builtin_nontemporal_store(o4, reinterpret_cast<f32x4_t *>(dst2));
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < g.N) dst2[e] = w[e];
                    }
                } else if (dgelu) {
                    // C = product * gelu'(z + bias), z the saved pre-activation laid out like C
                    const float *zp = g.aux_in + (int64_t)batch * g.c_bs + (int64_t)row * ldc + col;
                    float z[4] = {0.f, 0.f, 0.f, 0.f};
                    if (zvec) {
                        z[0] = zpre[i][pass].x; z[1] = zpre[i][pass].y; z[2] = zpre[i][pass].z; z[3] = zpre[i][pass].w;
                    } else if (col + 3 < g.N) {
                        const float4 z4 = *reinterpret_cast<const float4 *>(zp);
                        z[0] = z4.x; z[1] = z4.y; z[2] = z4.z; z[3] = z4.w;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < g.N) z[e] = zp[e];
                    }
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] = col + e < g.N ? v[e] * gelu_tanh_grad(z[e] + bias4[e]) : 0.0f;
                        csum[e] += v[e];
                    }
                } else if (!partial) {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        v[e] += bias4[e];
                        if (g.epilogue == MNI_EPI_BIAS_RELU) v[e] = fmaxf(v[e], 0.0f);
                        else if (g.epilogue == MNI_EPI_BIAS_GELU) v[e] = gelu_tanh(v[e]);
                    }
                }
                if (vec_ok && col + 3 < g.N) {
                    if (!partial && g.accumulate) {
                        const float4 c = *reinterpret_cast<const float4 *>(dst);
                        v[0] += c.x; v[1] += c.y; v[2] += c.z; v[3] += c.w;
                    }
                    // streaming store: C is written once and not read again by this kernel, so
                    // it need not displace the operand panels in L2
                    typedef float f32x4_t __attribute__((ext_vector_type(4)));
                    const f32x4_t o4 = {v[0], v[1], v[2], v[3]};
                    __builtin_nontemporal_store(o4, reinterpret_cast<f32x4_t *>(dst));
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        if (col + e < g.N) dst[e] = (!partial && g.accumulate) ? v[e] + dst[e] : v[e];
                    }
                }
            }
        }
        wave_sync();
    };
    epilogue_strip(std::integral_constant<int, 0>());
    if constexpr (TM > 1) epilogue_strip(std::integral_constant<int, 1>());
    if constexpr (TM > 2) epilogue_strip(std::integral_constant<int, 2>());
    if constexpr (TM > 3) epilogue_strip(std::integral_constant<int, 3>());
    // (stream-K: the next segment's prologue writes LDS that other wavefronts' patches still occupy)
    if (SK) __syncthreads();
    if (dgelu && g.colsum_part) {
        // lanes that share columns (same lane % LANES_PER_ROW) are added by butterfly steps; strip
        // (batch, tile row, wm) owns one row of the partial matrix
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
            for (int off = LANES_PER_ROW; off < 64; off <<= 1) csum[e] += __shfl_xor(csum[e], off, 64);
        if (lane < LANES_PER_ROW) {
            float *cp = g.colsum_part + (((int64_t)batch * g.tiles_m + tm) * 2 + wm) * (int64_t)g.N;
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < g.N) cp[col + e] = csum[e];
        }
    }
    if (SK && role == ROLE_PART) {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wavefront's part of the tile has reached L2
        __syncthreads();
        if (tid == 0) g.sk_flags[bid] = g.sk_epoch;
    }
    if (!(fin >> 30)) break;
    } while (SK);  // segments
#undef g
}

template <int AMODE, int BMODE, int TM, int TN, bool SK>
__global__ __launch_bounds__(NTHREADS, (TM * TN >= 2 ? 2 : 4)) void gemm_mfma_kernel(const GemmLaunch launch_args) {
    (void)launch_args;
    __shared__ float4 lds[gemm_lds_slots<AMODE, BMODE, TM, TN>()];
    gemm_mfma_body<AMODE, BMODE, TM, TN, SK>((LaunchPtr)__builtin_amdgcn_kernarg_segment_ptr(), blockIdx.x, gridDim.x, lds);
}

// Two independent products in one launch, both on 64 x 64 tiles or both on 128 x 128 (T = 1, 2), one workgroup per
// tile and all of K: workgroups [0, wgs_lead) work on the product named by `lead` (wgs_lead = its tile count rounded
// up to a multiple of 8, so that the other product's numbering starts on XCD 0 as well; the padding workgroups
// leave at once), the rest on the other.  For the two backward products of a matmul
// (src/native/src/ops/matmul.rs:199-222): when each of them alone is about one tile per CU, together they give
// every SIMD a second wavefront; and whatever their size they share one launch, one ramp-up and one tail.  The
// product with the longer K leads, so that its long-lived workgroups are dealt first and the short ones fill in
// behind them.
struct GemmPairLaunch {
    GemmLaunch g[2];
    unsigned lead, wgs_lead, tiles0, tiles1;
    // The other product's workgroups: wgs_other of them, each working through `chunk` tiles one after the other (tiles w,
    // w + wgs_other, ...).  chunk > 1 when the lead's K is that many times the other's and the whole launch is resident
    // at once: every workgroup then has the same number of K steps before it, and which CU gets how many of the short
    // tiles is no longer left to the order in which workgroup slots happen to fall free (1024 tiles of K = 1024 behind
    // 256 of K = 4096 took 492 us on most launches and 546 on one in four; four short tiles per workgroup: every launch
    // the same).
    unsigned wgs_other, chunk;
    // Column sums that ride along (a Linear layer's bias gradient: the sums of the matrix both products read): cs_out[c] =
    // sum over r of cs_src[r, c] for a contiguous [cs_rows, cs_cols] matrix, by cs_wgs workgroups behind the products'
    // (0: none), PAIR_CS_COLS columns each.  Behind, because a workgroup ahead of the tiles would take a tile's place in
    // the first round on a machine the tiles fill exactly, and that tile would run alone at the end; at the end they
    // start as the first tiles finish and run in the raggedness of the launch's tail.
    const float *cs_src;
    float *cs_out;
    int cs_rows, cs_cols;
    unsigned cs_wgs;
};
typedef const GemmPairLaunch __attribute__((address_space(4))) *PairPtr;

constexpr int PAIR_CS_COLS = 8, PAIR_CS_GROUPS = 128, PAIR_CS_DEPTH = 8;
static_assert(NTHREADS == 2 * PAIR_CS_GROUPS && PAIR_CS_COLS == 8, "the column sums of a paired launch split 256 threads into 2 column quads x 128 row groups");

// Workgroup b of the column sums: thread (quad, group) adds rows group, group + 128, ... of its four columns (eight
// loads in flight), the groups are added in order through LDS.  cs_cols is a multiple of 4 and both pointers are
// 16-byte aligned (checked by the launcher).
__device__ __forceinline__ void pair_colsum_role(PairPtr pp, const unsigned b, float4 *__restrict__ lds) {
    const int tid = threadIdx.x, cq = tid & 1, rg = tid >> 1;
    const int rows = pp->cs_rows, cols = pp->cs_cols;
    const int col = (int)b * PAIR_CS_COLS + 4 * cq;
    float4 acc[PAIR_CS_DEPTH];
#pragma unroll
    for (int u = 0; u < PAIR_CS_DEPTH; ++u) acc[u] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (col < cols) {
        const float *__restrict__ p = pp->cs_src + col;
        int r = rg;
        for (; r + PAIR_CS_GROUPS * (PAIR_CS_DEPTH - 1) < rows; r += PAIR_CS_GROUPS * PAIR_CS_DEPTH) {
            float4 v[PAIR_CS_DEPTH];
#pragma unroll
            for (int u = 0; u < PAIR_CS_DEPTH; ++u) v[u] = *reinterpret_cast<const float4 *>(p + (int64_t)(r + PAIR_CS_GROUPS * u) * cols);
#pragma unroll
            for (int u = 0; u < PAIR_CS_DEPTH; ++u) { acc[u].x += v[u].x; acc[u].y += v[u].y; acc[u].z += v[u].z; acc[u].w += v[u].w; }
        }
        for (; r < rows; r += PAIR_CS_GROUPS) {
            const float4 v = *reinterpret_cast<const float4 *>(p + (int64_t)r * cols);
            acc[0].x += v.x; acc[0].y += v.y; acc[0].z += v.z; acc[0].w += v.w;
        }
    }
#pragma unroll
    for (int w = PAIR_CS_DEPTH / 2; w >= 1; w >>= 1)
#pragma unroll
        for (int u = 0; u < w; ++u) { acc[u].x += acc[u + w].x; acc[u].y += acc[u + w].y; acc[u].z += acc[u + w].z; acc[u].w += acc[u + w].w; }
    lds[tid] = acc[0];
    __syncthreads();
    if (tid < 2 && col < cols) {
        float4 t = lds[tid];
        for (int g = 1; g < PAIR_CS_GROUPS; ++g) {
            const float4 v = lds[2 * g + tid];
            t.x += v.x; t.y += v.y; t.z += v.z; t.w += v.w;
        }
        *reinterpret_cast<float4 *>(pp->cs_out + col) = t;
    }
}

// CHUNKED: the instantiation for chunk > 1 (a loop around the body; the plain one keeps the body's straight-line code)
template <int AM0, int BM0, int AM1, int BM1, int T, bool CHUNKED>
__global__ __launch_bounds__(NTHREADS, (T >= 2 ? 2 : 4)) void gemm_mfma_pair_kernel(const GemmPairLaunch pair_args) {
    (void)pair_args;
    PairPtr pp = (PairPtr)__builtin_amdgcn_kernarg_segment_ptr();
    constexpr int S0 = gemm_lds_slots<AM0, BM0, T, T>(), S1 = gemm_lds_slots<AM1, BM1, T, T>();
    static_assert(S0 >= NTHREADS && S1 >= NTHREADS, "the column sums park one float4 per thread");
    __shared__ float4 lds[S0 > S1 ? S0 : S1];
    const unsigned b = blockIdx.x, tile_wgs = pp->wgs_lead + pp->wgs_other;
    if (b >= tile_wgs) {
        pair_colsum_role(pp, b - tile_wgs, lds);
        return;
    }
    const bool in_lead = b < pp->wgs_lead;
    const unsigned wg = in_lead ? b : b - pp->wgs_lead;
    const unsigned which = in_lead ? pp->lead : 1u - pp->lead;
    if constexpr (!CHUNKED) {
        if (which == 0) {
            if (wg < pp->tiles0) gemm_mfma_body<AM0, BM0, T, T, false>(&pp->g[0], wg, pp->tiles0, lds);
        } else {
            if (wg < pp->tiles1) gemm_mfma_body<AM1, BM1, T, T, false>(&pp->g[1], wg, pp->tiles1, lds);
        }
    } else {
        const unsigned reps = in_lead ? 1u : pp->chunk, stride = pp->wgs_other;
        if (which == 0) {
            for (unsigned rep = 0; rep < reps; ++rep) {
                const unsigned w = wg + rep * stride;
                if (w < pp->tiles0) gemm_mfma_body<AM0, BM0, T, T, false, true>(&pp->g[0], w, pp->tiles0, lds);
                if (rep + 1 < reps) __syncthreads();  // (the next tile's prologue writes LDS that this one's epilogue still reads)
            }
        } else {
            for (unsigned rep = 0; rep < reps; ++rep) {
                const unsigned w = wg + rep * stride;
                if (w < pp->tiles1) gemm_mfma_body<AM1, BM1, T, T, false, true>(&pp->g[1], w, pp->tiles1, lds);
                if (rep + 1 < reps) __syncthreads();
            }
        }
    }
}

// Workgroups of a stream-K instantiation that fit one CU together, by the runtime's occupancy calculation (asked once).
template <int AM, int BMO, int TM, int TN>
static int streamk_occupancy() {
    static int n = -1;
    if (n < 0) {
        int v = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&v, gemm_mfma_kernel<AM, BMO, TM, TN, true>, NTHREADS, 0) != hipSuccess) {
            (void)hipGetLastError();
            v = 0;
        }
        n = v;
    }
    return n;
}

template <int TM, int TN>
static int launch_modes(const GemmLaunch &g, int amode, int bmode, dim3 grid) {
    dim3 block(NTHREADS);
    hipStream_t s = ctx().stream;
    // A stream-K finisher waits for partial tiles of other workgroups of its XCD: the whole grid must be resident
    // at once.  The planner sizes it by gemm_mfma_resident_per_cu; here that figure is held against what the
    // runtime says about the instantiation that is about to run.
    const int cus_per_xcd = g.streamk && g.sk_xcds > 0 ? (ctx().compute_units > 0 ? ctx().compute_units : 256) / g.sk_xcds : 0;
#define MNI_LAUNCH(AM, BMO)                                                                        \
    do {                                                                                           \
        if (g.streamk) {                                                                           \
            if ((int64_t)streamk_occupancy<AM, BMO, TM, TN>() * cus_per_xcd < g.sk_wpx)           \
                return set_error(MNI_ERR_INVALID, "sgemm: stream-K grid of %d workgroups per XCD, but %d fit a CU", g.sk_wpx, \
                                 streamk_occupancy<AM, BMO, TM, TN>());                           \
            MNI_KERNEL_LAUNCH((gemm_mfma_kernel<AM, BMO, TM, TN, true>), grid, block, 0, s, g);   \
        } else MNI_KERNEL_LAUNCH((gemm_mfma_kernel<AM, BMO, TM, TN, false>), grid, block, 0, s, g);            \
    } while (0)
    if (amode == 2 || bmode == 2) MNI_LAUNCH(2, 2);
    else if (amode == 0 && bmode == 0) MNI_LAUNCH(0, 0);
    else if (amode == 0 && bmode == 1) MNI_LAUNCH(0, 1);
    else if (amode == 1 && bmode == 0) MNI_LAUNCH(1, 0);
    else MNI_LAUNCH(1, 1);
#undef MNI_LAUNCH
    return MNI_OK;
}

// tile_m / tile_n: 128 or 64 (g.tiles_m / g.tiles_n must be counted in those units)
int launch_gemm_mfma(const GemmLaunch &g, int amode, int bmode, int tile_m, int tile_n) {
    if ((int64_t)g.tiles_m * g.tiles_n * g.batch <= 0) return MNI_OK;
    if (g.streamk) {
        // what the kernel's arithmetic assumes about its grid and buffers
        if (g.split_k != 1 || g.sk_xcds < 1 || g.sk_wpx < 1 || g.sk_wpx > NTHREADS || !g.ws || !g.sk_flags || !g.status)
            return set_error(MNI_ERR_INVALID, "sgemm: inconsistent stream-K launch");
    }
    const int64_t blocks = g.streamk ? (int64_t)g.sk_xcds * g.sk_wpx : (int64_t)g.tiles_m * g.tiles_n * g.batch * g.split_k;
    if (blocks > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "sgemm: too many tiles (%lld)", (long long)blocks);
    dim3 grid((unsigned)blocks);
    int rc;
    if (tile_m == 128 && tile_n == 128) rc = launch_modes<2, 2>(g, amode, bmode, grid);
    else if (tile_m == 128 && tile_n == 64) rc = launch_modes<2, 1>(g, amode, bmode, grid);
    else if (tile_m == 64 && tile_n == 128) rc = launch_modes<1, 2>(g, amode, bmode, grid);
    else if (tile_m == 64 && tile_n == 64) rc = launch_modes<1, 1>(g, amode, bmode, grid);
    else return set_error(MNI_ERR_INVALID, "sgemm: unsupported tile %d x %d", tile_m, tile_n);
    MNI_TRY(rc);
    return check_launch("gemm_mfma_kernel");
}

// The product pairs a matmul backward gives rise to: product 0 has dC (row-major) as its A, product 1 has dC as
// its B; tiles of `tile` x `tile` (64 or 128; g.tiles_m / g.tiles_n count those), one workgroup per tile, all of K.
bool gemm_mfma_pair_eligible(int amode0, int bmode0, int amode1, int bmode1) {
    return amode0 == 0 && bmode0 <= 1 && amode1 <= 1 && bmode1 == 1;
}

template <int T, bool CHUNKED>
static void launch_pair_modes(const GemmPairLaunch &p, int bmode0, int amode1, dim3 grid) {
    const dim3 block(NTHREADS);
    hipStream_t s = ctx().stream;
    if (bmode0 == 0 && amode1 == 0) MNI_KERNEL_LAUNCH((gemm_mfma_pair_kernel<0, 0, 0, 1, T, CHUNKED>), grid, block, 0, s, p);
    else if (bmode0 == 0 && amode1 == 1) MNI_KERNEL_LAUNCH((gemm_mfma_pair_kernel<0, 0, 1, 1, T, CHUNKED>), grid, block, 0, s, p);
    else if (bmode0 == 1 && amode1 == 0) MNI_KERNEL_LAUNCH((gemm_mfma_pair_kernel<0, 1, 0, 1, T, CHUNKED>), grid, block, 0, s, p);
    else MNI_KERNEL_LAUNCH((gemm_mfma_pair_kernel<0, 1, 1, 1, T, CHUNKED>), grid, block, 0, s, p);
}

bool gemm_mfma_pair_takes_colsum(const PairColsum &cs) {
    return cs.src && cs.out && cs.rows > 0 && cs.cols > 0 && cs.cols % 4 == 0 && cs.rows <= 0x7fffffffLL && cs.cols <= (1LL << 24) &&
           ((uintptr_t)cs.src & 15) == 0 && ((uintptr_t)cs.out & 15) == 0;
}

int launch_gemm_mfma_pair(const GemmLaunch &g0, int amode0, int bmode0, const GemmLaunch &g1, int amode1, int bmode1, int tile,
                          const PairColsum *colsum) {
    if (!gemm_mfma_pair_eligible(amode0, bmode0, amode1, bmode1))
        return set_error(MNI_ERR_INVALID, "sgemm: product pair not eligible for the paired tile kernel");
    if (tile != 64 && tile != 128) return set_error(MNI_ERR_INVALID, "sgemm: paired tile kernel takes tiles of 64 or 128");
    if (colsum && !gemm_mfma_pair_takes_colsum(*colsum))
        return set_error(MNI_ERR_INVALID, "sgemm: the paired tile kernel's column sums take a 16-byte aligned matrix of a multiple of 4 columns");
    const int64_t t0 = (int64_t)g0.tiles_m * g0.tiles_n * g0.batch, t1 = (int64_t)g1.tiles_m * g1.tiles_n * g1.batch;
    if (g0.tiles_m != (g0.M + tile - 1) / tile || g0.tiles_n != (g0.N + tile - 1) / tile || g1.tiles_m != (g1.M + tile - 1) / tile ||
        g1.tiles_n != (g1.N + tile - 1) / tile || t0 <= 0 || t1 <= 0 || t0 + t1 + (1LL << 22) > 0x7fffffffLL || g0.split_k != 1 || g1.split_k != 1 ||
        g0.streamk || g1.streamk || g0.K <= 0 || g1.K <= 0 || g0.k_per_slice < g0.K || g1.k_per_slice < g1.K)
        return set_error(MNI_ERR_INVALID, "sgemm: paired tile kernel launched with a wrong plan");
    GemmPairLaunch p;
    p.g[0] = g0;
    p.g[1] = g1;
    p.tiles0 = (unsigned)t0;
    p.tiles1 = (unsigned)t1;
    p.lead = g1.K > g0.K ? 1u : 0u;
    p.wgs_lead = (unsigned)(((p.lead ? t1 : t0) + 7) / 8 * 8);
    {
        const int64_t k_lead = p.lead ? g1.K : g0.K, k_other = p.lead ? g0.K : g1.K, t_other = p.lead ? t0 : t1;
        const int64_t c = k_lead / k_other;
        const int64_t slots = (int64_t)(ctx().compute_units > 0 ? ctx().compute_units : 256) * gemm_mfma_resident_per_cu(tile, tile);
        const bool even = c >= 2 && c <= 8 && t_other % c == 0 && (t_other / c) % 8 == 0 && (int64_t)p.wgs_lead + t_other / c <= slots;
        p.chunk = even ? (unsigned)c : 1u;
        p.wgs_other = (unsigned)(t_other / p.chunk);
    }
    p.cs_src = colsum ? colsum->src : nullptr;
    p.cs_out = colsum ? colsum->out : nullptr;
    p.cs_rows = colsum ? (int)colsum->rows : 0;
    p.cs_cols = colsum ? (int)colsum->cols : 0;
    p.cs_wgs = colsum ? (unsigned)((colsum->cols + PAIR_CS_COLS - 1) / PAIR_CS_COLS) : 0u;   // (at most 2^21)
    const dim3 grid(p.wgs_lead + p.wgs_other + p.cs_wgs);
    if (tile == 128 && p.chunk > 1) launch_pair_modes<2, true>(p, bmode0, amode1, grid);
    else if (tile == 128) launch_pair_modes<2, false>(p, bmode0, amode1, grid);
    else if (p.chunk > 1) launch_pair_modes<1, true>(p, bmode0, amode1, grid);
    else launch_pair_modes<1, false>(p, bmode0, amode1, grid);
    return check_launch("gemm_mfma_pair_kernel");
}

int gemm_mfma_tile_k() { return BK; }
// 128-wide tiles: two waves per SIMD by registers (and two tiles' LDS); 64 x 64: four.
int gemm_mfma_resident_per_cu(int tile_m, int tile_n) { return tile_m * tile_n > 64 * 64 ? 2 : 4; }

}  // namespace mni
