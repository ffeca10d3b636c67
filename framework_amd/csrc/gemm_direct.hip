// Batched products of many small output tiles on the MFMA matrix cores, with
// the operands taken from memory straight into the registers the matrix
// instruction reads -- no LDS staging, no barrier in the K loop.
//
//   C[b] = epilogue( op(A)[b] (M x K)  *  op(B)[b] (K x N) )
//
// What this form is for.  The tile kernel (gemm_mfma.hip) is built around a
// long K loop over a few hundred resident tiles: two LDS stages, one K step of
// 32 requested ahead, a barrier per step.  The batched products of an
// attention layer (reference call sites: src/native/src/ops/matmul.rs:54-70
// with a permuted operand from ops/layout.rs:112-134, and the two backward
// products of ops/matmul.rs:199-222) are a different animal:
//   * scores  S[b] = Q[b] K[b]^T : thousands of 64 x 64 tiles with K = 64 (two K
//     steps: all prologue and epilogue, no loop to speak of), output-bound;
//   * dQ[b] = dS[b] K[b],  dK[b]^T = Q[b]^T dS[b] : a few hundred 64 x 64 tiles that
//     each stream a long, thin operand once from HBM -- with one workgroup per
//     CU and 16 KB requested ahead the memory system idles most of the time.
// Here every wavefront requests everything it will need for up to 128 K
// values (64 KB per wavefront, 256 KB per CU in flight) before its first
// MFMA, and the MFMAs then run down the registers as the data arrives.
//
// Work split.  A workgroup owns one 64 x 64 tile of C.  KSPLIT = 1: the
// workgroup is a single wavefront that contracts all of K and stores its
// accumulators straight from registers.  KSPLIT = 4: four wavefronts take a
// quarter of K each, all four hold a full 64 x 64 partial tile, and the
// partials are added in wavefront order through LDS (fixed order: the result
// depends on the shape only), which also turns them into 16-byte row stores.
//
// Register layout.  v_mfma_f32_32x32x2_f32 takes A[i = lane % 32][k = lane / 32]
// and B[k = lane / 32][j = lane % 32], one float each.  Let i = lane % 32 and
// h = lane / 32; MFMA j of chunk c (8 K values per chunk) contracts
// k = 8c + 4h + j.
//   * an operand with unit stride along K (mode 0) is read with one 16-byte
//     load per lane, row and chunk: lane (i, h) holds k = 8c + 4h .. + 3 of
//     row 32 blk + i -- exactly the four values it feeds to MFMAs j = 0..3;
//   * an operand with unit stride along M / N (mode 1) is read with one 8-byte
//     load per lane and K row: lane (i, h) holds elements 2i and 2i + 1 of row
//     k = 8c + 4h + j, so the two 32-wide MFMA blocks of the tile side take
//     the even and the odd rows / columns (a permutation that the epilogue
//     undoes by construction).  A half wavefront reads 256 contiguous bytes.
// Rows beyond an edge re-read the last valid row (or row pair) and land in
// accumulator rows / columns that are never stored; K beyond its end reads as
// zero (guarded loads, in a last partial phase only).
#include "common.h"
#include "gemm_internal.h"

namespace mni {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

static constexpr int DT = 64;        // tile side
static constexpr int DPHASE = 32;    // K values per phase (4 chunks of 8)
static constexpr int DPITCH = DT + 4;  // LDS row pitch of a partial tile, in floats

__device__ __forceinline__ float dk_gelu(float x) {
    // tanh-approximation GELU of the reference (src/native/src/ops/activation.rs:15-18)
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}

__device__ __forceinline__ float dk_pick(const f32x4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }

// One phase (32 K values) of one operand's 64-wide tile side, as a lane holds it.
template <int MODE> struct PhaseRegs;
template <> struct PhaseRegs<0> { f32x4 v[2][4]; };  // [block][chunk]: k = 8c + 4h + component
template <> struct PhaseRegs<1> { f32x2 v[4][4]; };  // [chunk][j]: k = 8c + 4h + j; x = block 0, y = block 1

__device__ __forceinline__ float operand_of(const PhaseRegs<0> &r, int blk, int c, int j) { return dk_pick(r.v[blk][c], j); }
__device__ __forceinline__ float operand_of(const PhaseRegs<1> &r, int blk, int c, int j) { return blk == 0 ? r.v[c][j].x : r.v[c][j].y; }

// Where a lane's loads of one operand start.  Mode 0: p[blk] = first K value
// of row (32 blk + i, clamped to the edge) plus 4h.  Mode 1: p[0] = element
// (2i, clamped) of K row 4h; `ld` is the stride between K rows.
template <int MODE> struct OperandPtr {
    const float *p[2];
    int64_t ld;
};

template <int MODE>
__device__ __forceinline__ OperandPtr<MODE> operand_ptr(const float *base, int64_t mn_stride, int64_t k_stride, int mn0,
                                                        int mn_extent, int i, int h) {
    OperandPtr<MODE> o;
    if (MODE == 0) {
        // k_stride == 1
        o.p[0] = base + (int64_t)min(mn0 + i, mn_extent - 1) * mn_stride + 4 * h;
        o.p[1] = base + (int64_t)min(mn0 + 32 + i, mn_extent - 1) * mn_stride + 4 * h;
        o.ld = mn_stride;
    } else {
        // mn_stride == 1, mn_extent even
        o.p[0] = base + min(mn0 + 2 * i, mn_extent - 2) + (int64_t)(4 * h) * k_stride;
        o.p[1] = o.p[0];
        o.ld = k_stride;
    }
    return o;
}

// Full phase starting at K index k0 (relative to the operand's first K value): no guards.
__device__ __forceinline__ void load_phase(PhaseRegs<0> &r, const OperandPtr<0> &o, int k0) {
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int c = 0; c < 4; ++c) r.v[b][c] = *reinterpret_cast<const f32x4 *>(o.p[b] + k0 + 8 * c);
}
__device__ __forceinline__ void load_phase(PhaseRegs<1> &r, const OperandPtr<1> &o, int k0) {
    const float *p = o.p[0] + (int64_t)k0 * o.ld;
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int j = 0; j < 4; ++j) r.v[c][j] = *reinterpret_cast<const f32x2 *>(p + (int64_t)(8 * c + j) * o.ld);
}
// Partial phase: K values at or beyond k_end read as zero (k_end is a multiple
// of 4 for a mode-0 operand, so a 16-byte piece is either whole or absent).
__device__ __forceinline__ void load_phase_guarded(PhaseRegs<0> &r, const OperandPtr<0> &o, int k0, int k_end, int h) {
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const bool ok = k0 + 8 * c + 4 * h < k_end;
            r.v[b][c] = ok ? *reinterpret_cast<const f32x4 *>(o.p[b] + k0 + 8 * c) : f32x4{0.f, 0.f, 0.f, 0.f};
        }
}
__device__ __forceinline__ void load_phase_guarded(PhaseRegs<1> &r, const OperandPtr<1> &o, int k0, int k_end, int h) {
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int k = k0 + 8 * c + j;
            const bool ok = k + 4 * h < k_end;
            r.v[c][j] = ok ? *reinterpret_cast<const f32x2 *>(o.p[0] + (int64_t)k * o.ld) : f32x2{0.f, 0.f};
        }
}

template <int AMODE, int BMODE>
__device__ __forceinline__ void mfma_phase(floatx16 (&acc)[2][2], const PhaseRegs<AMODE> &ra, const PhaseRegs<BMODE> &rb) {
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int q = 0; q < 2; ++q)
                    acc[a][q] = __builtin_amdgcn_mfma_f32_32x32x2f32(operand_of(ra, a, c, j), operand_of(rb, q, c, j), acc[a][q], 0, 0, 0);
}

// Row of the tile that index `idx` (0..31) of block `blk` stands for.
template <int MODE> __device__ __forceinline__ int tile_index(int blk, int idx) { return MODE == 0 ? 32 * blk + idx : 2 * idx + blk; }

// NPH > 0: every wavefront has exactly NPH full phases and nothing else; all
// of them are requested before the first MFMA.  NPH = 0: any K; two phases in
// flight, a guarded phase for what is left.
template <int AMODE, int BMODE, int KSPLIT, int NPH>
__global__ __launch_bounds__(64 * KSPLIT, (KSPLIT == 1 || NPH == 0) ? 2 : 1) void gemm_direct_kernel(const GemmLaunch g) {
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = KSPLIT > 1 ? __builtin_amdgcn_readfirstlane(tid >> 6) : 0;
    const int i = lane & 31, h = lane >> 5;

    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2:
    // renumber so that every XCD works on one contiguous run of tiles (tiles
    // of one batch share their operand panels).
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
    const int m0 = tm * DT, n0 = tn * DT;

    // this wavefront's K range: whole phases, dealt in wavefront order
    int kb = 0, ke = g.K;
    if (KSPLIT > 1) {
        const int phases = (g.K + DPHASE - 1) / DPHASE;
        const int per = (phases + KSPLIT - 1) / KSPLIT;
        kb = min(g.K, wave * per * DPHASE);
        ke = min(g.K, kb + per * DPHASE);
    }

    const float *Ab = g.A + (int64_t)(batch % g.a_bcount) * g.a_bs + (int64_t)kb * g.a_cs;
    const float *Bb = g.B + (int64_t)(batch % g.b_bcount) * g.b_bs + (int64_t)kb * g.b_rs;
    // op(A)(m, k): M stride a_rs, K stride a_cs.  op(B)(k, n): K stride b_rs, N stride b_cs.
    const OperandPtr<AMODE> pa = operand_ptr<AMODE>(Ab, g.a_rs, g.a_cs, m0, g.M, i, h);
    const OperandPtr<BMODE> pb = operand_ptr<BMODE>(Bb, g.b_cs, g.b_rs, n0, g.N, i, h);
    const int klen = ke - kb;

    floatx16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int q = 0; q < 2; ++q)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][q][e] = 0.0f;

    if (NPH > 0) {
        PhaseRegs<AMODE> ra[NPH > 0 ? NPH : 1];
        PhaseRegs<BMODE> rb[NPH > 0 ? NPH : 1];
#pragma unroll
        for (int s = 0; s < NPH; ++s) {
            load_phase(ra[s], pa, s * DPHASE);
            load_phase(rb[s], pb, s * DPHASE);
        }
        // Left alone, the instruction scheduler moves every load down to its
        // first use to save registers, and the kernel then waits for memory
        // once per load.  Requests first, arithmetic after.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < NPH; ++s) {
            mfma_phase<AMODE, BMODE>(acc, ra[s], rb[s]);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
        const int nfull = klen / DPHASE;
        if (nfull > 0) {
            // Two phases in flight.  Every load is unconditional (past the end
            // the last full phase is fetched again and not used), so that each
            // register buffer has one producer in the loop.
            PhaseRegs<AMODE> a0, a1;
            PhaseRegs<BMODE> b0, b1;
            load_phase(a0, pa, 0);
            load_phase(b0, pb, 0);
            load_phase(a1, pa, min(1, nfull - 1) * DPHASE);
            load_phase(b1, pb, min(1, nfull - 1) * DPHASE);
            // (the fences keep requests and arithmetic in this order: left alone, the
            // scheduler moves every load down to its first use to save registers)
            __builtin_amdgcn_sched_barrier(0);
            for (int p = 0; p < nfull; p += 2) {
                mfma_phase<AMODE, BMODE>(acc, a0, b0);
                __builtin_amdgcn_sched_barrier(0);
                load_phase(a0, pa, min(p + 2, nfull - 1) * DPHASE);
                load_phase(b0, pb, min(p + 2, nfull - 1) * DPHASE);
                __builtin_amdgcn_sched_barrier(0);
                if (p + 1 < nfull) mfma_phase<AMODE, BMODE>(acc, a1, b1);
                __builtin_amdgcn_sched_barrier(0);
                load_phase(a1, pa, min(p + 3, nfull - 1) * DPHASE);
                load_phase(b1, pb, min(p + 3, nfull - 1) * DPHASE);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (nfull * DPHASE < klen) {
            PhaseRegs<AMODE> a0;
            PhaseRegs<BMODE> b0;
            load_phase_guarded(a0, pa, nfull * DPHASE, klen, h);
            load_phase_guarded(b0, pb, nfull * DPHASE, klen, h);
            mfma_phase<AMODE, BMODE>(acc, a0, b0);
        }
    }

    // ---- epilogue ---------------------------------------------------------------
    // acc[a][q][e] of lane (i, h) is C[tile row tile_index<AMODE>(a, 8 (e / 4) + 4 h + e % 4)]
    //                                 [tile col tile_index<BMODE>(q, i)].
    float *Cb = g.C + (int64_t)batch * g.c_bs;
    auto finish = [&](float v, int col) {
        if (g.epilogue != MNI_EPI_NONE) {
            v += g.bias[col];
            if (g.epilogue == MNI_EPI_BIAS_RELU) v = fmaxf(v, 0.0f);
            else if (g.epilogue == MNI_EPI_BIAS_GELU) v = dk_gelu(v);
        }
        return v;
    };
    if (KSPLIT == 1) {
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = m0 + tile_index<AMODE>(a, 8 * (e >> 2) + 4 * h + (e & 3));
                if (row >= g.M) continue;
                float *dst = Cb + (int64_t)row * g.ldc;
                if (BMODE == 0) {
#pragma unroll
                    for (int q = 0; q < 2; ++q) {
                        const int col = n0 + 32 * q + i;
                        if (col < g.N) {
                            float v = finish(acc[a][q][e], col);
                            if (g.accumulate) v += dst[col];
                            __builtin_nontemporal_store(v, dst + col);
                        }
                    }
                } else {
                    const int col = n0 + 2 * i;  // N is even
                    if (col < g.N) {
                        f32x2 v = {finish(acc[a][0][e], col), finish(acc[a][1][e], col + 1)};
                        if (g.accumulate) v += *reinterpret_cast<const f32x2 *>(dst + col);
                        __builtin_nontemporal_store(v, reinterpret_cast<f32x2 *>(dst + col));
                    }
                }
            }
    } else {
        __shared__ float red[KSPLIT > 1 ? KSPLIT : 1][DT][DPITCH];
#pragma unroll
        for (int a = 0; a < 2; ++a)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int rowl = tile_index<AMODE>(a, 8 * (e >> 2) + 4 * h + (e & 3));
                if (BMODE == 0) {
                    red[wave][rowl][i] = acc[a][0][e];
                    red[wave][rowl][32 + i] = acc[a][1][e];
                } else {
                    *reinterpret_cast<f32x2 *>(&red[wave][rowl][2 * i]) = f32x2{acc[a][0][e], acc[a][1][e]};
                }
            }
        __syncthreads();
        // 64 x 64 outputs, 256 threads: four 16-byte pieces each, the partials added in wavefront order
        constexpr int PIECES = DT * DT / 4 / (64 * KSPLIT);
#pragma unroll
        for (int p = 0; p < PIECES; ++p) {
            const int rowl = tid / 16 + (64 * KSPLIT / 16) * p, coll = 4 * (tid % 16);
            f32x4 s = *reinterpret_cast<const f32x4 *>(&red[0][rowl][coll]);
#pragma unroll
            for (int w = 1; w < KSPLIT; ++w) s += *reinterpret_cast<const f32x4 *>(&red[w][rowl][coll]);
            const int row = m0 + rowl, col = n0 + coll;
            if (row >= g.M || col >= g.N) continue;
            float *dst = Cb + (int64_t)row * g.ldc + col;
            float v[4] = {s.x, s.y, s.z, s.w};
            if (col + 3 < g.N) {
#pragma unroll
                for (int x = 0; x < 4; ++x) v[x] = finish(v[x], col + x);
                f32x4 o = {v[0], v[1], v[2], v[3]};
                if (g.accumulate) o += *reinterpret_cast<const f32x4 *>(dst);
                __builtin_nontemporal_store(o, reinterpret_cast<f32x4 *>(dst));
            } else {
#pragma unroll
                for (int x = 0; x < 4; ++x)
                    if (col + x < g.N) {
                        const float o = finish(v[x], col + x);
                        dst[x] = g.accumulate ? o + dst[x] : o;
                    }
            }
        }
    }
}

// Operand layouts this form reads: both K-contiguous or M/N-contiguous;
// 16-byte pieces along K need K % 4 == 0, 8-byte pieces along M / N an even
// extent.  (Any 4-byte aligned address will do for either.)
bool gemm_direct_eligible(const GemmLaunch &g, int amode, int bmode) {
    if (g.K <= 0 || amode > 1 || bmode > 1) return false;
    if ((amode == 0 || bmode == 0) && g.K % 4 != 0) return false;
    if (amode == 1 && g.M % 2 != 0) return false;
    if (bmode == 1 && g.N % 2 != 0) return false;
    return true;
}

template <int AMODE, int BMODE>
static void launch_direct_modes(const GemmLaunch &g, int ksplit, dim3 grid) {
    hipStream_t s = ctx().stream;
    if (ksplit == 1) {
        if (g.K == 2 * DPHASE) MNI_KERNEL_LAUNCH((gemm_direct_kernel<AMODE, BMODE, 1, 2>), grid, dim3(64), 0, s, g);
        else MNI_KERNEL_LAUNCH((gemm_direct_kernel<AMODE, BMODE, 1, 0>), grid, dim3(64), 0, s, g);
    } else {
        if (g.K == 4 * 4 * DPHASE) MNI_KERNEL_LAUNCH((gemm_direct_kernel<AMODE, BMODE, 4, 4>), grid, dim3(256), 0, s, g);
        else MNI_KERNEL_LAUNCH((gemm_direct_kernel<AMODE, BMODE, 4, 0>), grid, dim3(256), 0, s, g);
    }
}

// g.tiles_m / g.tiles_n must count 64 x 64 tiles; ksplit is 1 or 4.
int launch_gemm_direct(const GemmLaunch &g, int amode, int bmode, int ksplit) {
    if (!gemm_direct_eligible(g, amode, bmode)) return set_error(MNI_ERR_INVALID, "sgemm: operand layout not eligible for the direct kernel");
    if (ksplit != 1 && ksplit != 4) return set_error(MNI_ERR_INVALID, "sgemm: direct kernel takes 1 or 4 K parts, got %d", ksplit);
    if (g.tiles_m != (g.M + DT - 1) / DT || g.tiles_n != (g.N + DT - 1) / DT)
        return set_error(MNI_ERR_INVALID, "sgemm: direct kernel launched with a wrong tile count");
    const int64_t blocks = (int64_t)g.tiles_m * g.tiles_n * g.batch;
    if (blocks <= 0) return MNI_OK;
    if (blocks > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "sgemm: too many tiles (%lld)", (long long)blocks);
    const dim3 grid((unsigned)blocks);
    if (amode == 0 && bmode == 0) launch_direct_modes<0, 0>(g, ksplit, grid);
    else if (amode == 0 && bmode == 1) launch_direct_modes<0, 1>(g, ksplit, grid);
    else if (amode == 1 && bmode == 0) launch_direct_modes<1, 0>(g, ksplit, grid);
    else launch_direct_modes<1, 1>(g, ksplit, grid);
    return check_launch("gemm_direct_kernel");
}

}  // namespace mni
