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
// blocks of v_mfma_f32_32x32x2_f32 (16 accumulator VGPRs per block).  Tiles are
// staged through LDS, double-buffered, one barrier per K step: while the MFMAs
// of step t run out of LDS stage t&1, the global loads of step t+1 are in
// flight into registers and are written to the other stage afterwards.
//
// LDS layout.  Both operand tiles are stored "K-quad major":
//     tile[k/4][row][k%4]        (row = m for A, n for B; one float4 per row)
// so that one ds_read_b128 gives a lane the four K values it feeds to four
// consecutive MFMAs, and the 32 lanes of a half-wave read 32 consecutive
// float4 (conflict-free).  The MFMA takes k = lane/32 from each lane; because
// A and B use the same (k/4, k%4) split, lane half h contracts k = 8c+4h+j at
// MFMA j of chunk c, and the order of the K sum is the only thing that differs
// from a textbook loop.
//
// Operand layouts (transposes folded into the load path).  An operand whose K
// axis has unit stride (A row-major, or B given as its transpose) is loaded
// with 16-byte loads along K and stored to LDS as is.  An operand whose M/N
// axis has unit stride (B row-major, or A given as its transpose) is loaded as
// a 4(k) x 4(mn) micro-tile with 16-byte loads along M/N and transposed in
// registers on the way to LDS.  Anything else (arbitrary strides, unaligned
// bases, edge tiles) takes guarded scalar loads into the same register layout.
#include "common.h"
#include "gemm_internal.h"

namespace mni {

typedef float floatx16 __attribute__((ext_vector_type(16)));

static constexpr int BM = 128, BN = 128, BK = 32;
static constexpr int KQ = BK / 4;           // K quads per tile
static constexpr int PAD = 2;               // float4 of padding per K-quad slice
static constexpr int SLICE = BM + PAD;      // float4 per K-quad slice
static constexpr int NTHREADS = 256;

// Row r of a tile sits at float4 slot r ^ ((r >> 4) & 3) of its K-quad slice.
// Within an aligned group of 16 rows this is a permutation, so the MFMA operand
// reads (16 consecutive rows per LDS pass) stay conflict-free; it spreads the
// 16 rows 4*j + i that the micro-tile stores write in one pass over all 16
// bank groups (they would otherwise collide four ways).
__device__ __forceinline__ int lds_row(int r) { return r ^ ((r >> 4) & 3); }

// ---- global -> register loads ---------------------------------------------
// Register layout LAYOUT 0 (K contiguous): thread owns float4 #(tid + 256 i),
//   i = 0..3, where float4 #f is row f/8, K quad f%8.
// Register layout LAYOUT 1 (M/N contiguous): thread owns the 4 x 4 micro-tile
//   rows 4*(tid%32)..+3, K quad tid/32; v[j] holds k = 4*quad + j across the
//   four rows.

template <int LAYOUT>
__device__ __forceinline__ void load_fast(const float *__restrict__ p, int64_t ld, int tid, float4 (&v)[4]) {
    if (LAYOUT == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int f = tid + NTHREADS * i;
            int row = f >> 3, q = f & 7;
            v[i] = *reinterpret_cast<const float4 *>(p + (int64_t)row * ld + 4 * q);
        }
    } else {
        int r4 = tid & 31, q = tid >> 5;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            v[j] = *reinterpret_cast<const float4 *>(p + 4 * r4 + (int64_t)(4 * q + j) * ld);
    }
}

// Guarded element-wise load: element (row, k) lives at p[row * rs + k * cs];
// rows >= rmax or k >= kmax read as zero.
template <int LAYOUT>
__device__ __forceinline__ void load_guarded(const float *__restrict__ p, int64_t rs, int64_t cs, int rmax,
                                             int kmax, int tid, float4 (&v)[4]) {
    if (LAYOUT == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int f = tid + NTHREADS * i;
            int row = f >> 3, q = f & 7;
            float t[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                int k = 4 * q + e;
                t[e] = (row < rmax && k < kmax) ? p[(int64_t)row * rs + (int64_t)k * cs] : 0.0f;
            }
            v[i] = make_float4(t[0], t[1], t[2], t[3]);
        }
    } else {
        int r4 = tid & 31, q = tid >> 5;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int k = 4 * q + j;
            float t[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                int row = 4 * r4 + e;
                t[e] = (row < rmax && k < kmax) ? p[(int64_t)row * rs + (int64_t)k * cs] : 0.0f;
            }
            v[j] = make_float4(t[0], t[1], t[2], t[3]);
        }
    }
}

// ---- register -> LDS --------------------------------------------------------
template <int LAYOUT>
__device__ __forceinline__ void store_lds(float4 *__restrict__ tile, int tid, const float4 (&v)[4]) {
    if (LAYOUT == 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            int f = tid + NTHREADS * i;
            int row = f >> 3, q = f & 7;
            tile[q * SLICE + lds_row(row)] = v[i];
        }
    } else {
        int r4 = tid & 31, q = tid >> 5;
        tile[q * SLICE + lds_row(4 * r4 + 0)] = make_float4(v[0].x, v[1].x, v[2].x, v[3].x);
        tile[q * SLICE + lds_row(4 * r4 + 1)] = make_float4(v[0].y, v[1].y, v[2].y, v[3].y);
        tile[q * SLICE + lds_row(4 * r4 + 2)] = make_float4(v[0].z, v[1].z, v[2].z, v[3].z);
        tile[q * SLICE + lds_row(4 * r4 + 3)] = make_float4(v[0].w, v[1].w, v[2].w, v[3].w);
    }
}

__device__ __forceinline__ float gelu_tanh(float x) {
    // tanh-approximation GELU of the reference (src/native/src/ops/activation.rs:15-18)
    const float s = 0.7978845608028654f;  // sqrt(2/pi)
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}

// MODE: 0 = K axis contiguous + 16-byte aligned, 1 = M/N axis contiguous +
// aligned, 2 = arbitrary strides (always guarded scalar loads, layout 0).
template <int AMODE, int BMODE>
__global__ __launch_bounds__(NTHREADS, 2) void gemm_mfma_kernel(const GemmLaunch g) {
    constexpr int AL = AMODE == 1 ? 1 : 0;
    constexpr int BL = BMODE == 1 ? 1 : 0;
    __shared__ float4 lds[2][2][KQ * SLICE];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- workgroup -> (tile, batch, slice) ---------------------------------
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.
    // Renumber so that every XCD works on one contiguous run of tiles, then
    // walk tiles in column-grouped order so concurrently resident tiles share
    // A row panels and B column panels in that L2.
    int64_t pid = blockIdx.x;
    {
        const int64_t total = gridDim.x;
        const int64_t q = total >> 3, r = total & 7;
        const int64_t x = pid & 7, i = pid >> 3;
        pid = (x < r ? x * (q + 1) : r * (q + 1) + (x - r) * q) + i;
    }
    const int tiles = g.tiles_m * g.tiles_n;
    const int z = (int)(pid / tiles);
    int t = (int)(pid - (int64_t)z * tiles);
    const int batch = z / g.split_k;
    const int slice = z - batch * g.split_k;
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
    const int k_begin = slice * g.k_per_slice;
    const int k_end = min(g.K, k_begin + g.k_per_slice);
    const int klen = max(k_end - k_begin, 0);
    const int nkt = (klen + BK - 1) / BK;

    const float *__restrict__ Ap =
        g.A + (int64_t)(batch % g.a_bcount) * g.a_bs + (int64_t)m0 * g.a_rs + (int64_t)k_begin * g.a_cs;
    const float *__restrict__ Bp =
        g.B + (int64_t)(batch % g.b_bcount) * g.b_bs + (int64_t)n0 * g.b_cs + (int64_t)k_begin * g.b_rs;
    const int mrem = g.M - m0, nrem = g.N - n0;
    const bool a_full = AMODE != 2 && mrem >= BM;
    const bool b_full = BMODE != 2 && nrem >= BN;
    // leading dimension seen by the fast loaders
    const int64_t a_ld = AMODE == 0 ? g.a_rs : g.a_cs;
    const int64_t b_ld = BMODE == 0 ? g.b_cs : g.b_rs;

    floatx16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    float4 ra[4], rb[4];

    auto load_tiles = [&](int kt) {
        const int k0 = kt * BK;
        const int krem = klen - k0;
        // A tile: rows = m, element (m, k) at Ap[m * a_rs + k * a_cs]
        if (a_full && krem >= BK) {
            if (AMODE == 0) load_fast<0>(Ap + (int64_t)k0, a_ld, tid, ra);
            else load_fast<1>(Ap + (int64_t)k0 * a_ld, a_ld, tid, ra);
        } else {
            load_guarded<AL>(Ap + (int64_t)k0 * g.a_cs, g.a_rs, g.a_cs, mrem, krem, tid, ra);
        }
        // B tile: rows = n, element (n, k) at Bp[n * b_cs + k * b_rs]
        if (b_full && krem >= BK) {
            if (BMODE == 0) load_fast<0>(Bp + (int64_t)k0, b_ld, tid, rb);
            else load_fast<1>(Bp + (int64_t)k0 * b_ld, b_ld, tid, rb);
        } else {
            load_guarded<BL>(Bp + (int64_t)k0 * g.b_rs, g.b_cs, g.b_rs, nrem, krem, tid, rb);
        }
    };

    if (nkt > 0) {
        load_tiles(0);
        store_lds<AL>(lds[0][0], tid, ra);
        store_lds<BL>(lds[0][1], tid, rb);
    }
    __syncthreads();

    const int r = lane & 31, h = lane >> 5;
    // float4 slots of this lane's two A row blocks and two B column blocks
    const int a_row0 = lds_row(wm * 64 + r), a_row1 = lds_row(wm * 64 + 32 + r);
    const int b_row0 = lds_row(wn * 64 + r), b_row1 = lds_row(wn * 64 + 32 + r);
    constexpr int NCHUNK = KQ / 2;  // chunks of 8 K values: 16 MFMAs each

    // One chunk = 8 K values = 16 MFMAs in 4 groups of 4 (group j uses element
    // j of each operand float4).  The four ds_read_b128 of the NEXT chunk are
    // issued after the first three groups, and in the last chunk of a step the LDS
    // writes of the next stage take their place, so LDS traffic is spread under
    // the MFMAs instead of bunching up in front of a wait.  sched_barrier keeps
    // the compiler from regrouping them.
    float4 fa0, fa1, fb0, fb1;     // fragments in use
    float4 na0, na1, nb0, nb1;     // fragments of the next chunk
    auto mfma4 = [&](int j) {
        const float a0 = j == 0 ? fa0.x : j == 1 ? fa0.y : j == 2 ? fa0.z : fa0.w;
        const float a1 = j == 0 ? fa1.x : j == 1 ? fa1.y : j == 2 ? fa1.z : fa1.w;
        const float b0 = j == 0 ? fb0.x : j == 1 ? fb0.y : j == 2 ? fb0.z : fb0.w;
        const float b1 = j == 0 ? fb1.x : j == 1 ? fb1.y : j == 2 ? fb1.z : fb1.w;
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
    };

    for (int kt = 0; kt < nkt; ++kt) {
        const int cur = kt & 1;
        const bool more = kt + 1 < nkt;
        if (more) load_tiles(kt + 1);  // global loads of the next K step fly during this step's MFMAs

        const float4 *As = lds[cur][0], *Bs = lds[cur][1];
        fa0 = As[h * SLICE + a_row0]; fa1 = As[h * SLICE + a_row1];
        fb0 = Bs[h * SLICE + b_row0]; fb1 = Bs[h * SLICE + b_row1];
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) {
            const bool last = c == NCHUNK - 1;
            const int qn = (2 * (c + 1) + h) * SLICE;
            __builtin_amdgcn_sched_barrier(0);
            mfma4(0);
            __builtin_amdgcn_sched_barrier(0);
            if (!last) { na0 = As[qn + a_row0]; na1 = As[qn + a_row1]; }
            else if (more) store_lds<AL>(lds[cur ^ 1][0], tid, ra);
            __builtin_amdgcn_sched_barrier(0);
            mfma4(1);
            __builtin_amdgcn_sched_barrier(0);
            if (!last) nb0 = Bs[qn + b_row0];
            else if (more) store_lds<BL>(lds[cur ^ 1][1], tid, rb);
            __builtin_amdgcn_sched_barrier(0);
            mfma4(2);
            __builtin_amdgcn_sched_barrier(0);
            if (!last) nb1 = Bs[qn + b_row1];
            __builtin_amdgcn_sched_barrier(0);
            mfma4(3);
            __builtin_amdgcn_sched_barrier(0);
            if (!last) { fa0 = na0; fa1 = na1; fb0 = nb0; fb1 = nb1; }
        }
        __syncthreads();
    }

    // ---- epilogue -----------------------------------------------------------
    // A 32 x 32 MFMA block leaves lane l with column l%32 and rows
    // 8*(e/4) + 4*(l/32) + e%4, e = 0..15: each store instruction writes two
    // runs of 32 consecutive floats.
    float *__restrict__ Cb;
    int64_t ldc;
    const bool partial = g.split_k > 1;
    if (partial) {
        Cb = g.ws + ((int64_t)slice * g.batch + batch) * (int64_t)g.M * g.N;
        ldc = g.N;
    } else {
        Cb = g.C + (int64_t)batch * g.c_bs;
        ldc = g.ldc;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int col = n0 + wn * 64 + j * 32 + r;
        const bool col_ok = col < g.N;
        float bias = 0.0f;
        if (!partial && g.epilogue != MNI_EPI_NONE && col_ok) bias = g.bias[col];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int row_base = m0 + wm * 64 + i * 32 + 4 * h;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int row = row_base + 8 * (e >> 2) + (e & 3);
                if (col_ok && row < g.M) {
                    float v = acc[i][j][e];
                    float *dst = Cb + (int64_t)row * ldc + col;
                    if (!partial) {
                        v += bias;
                        if (g.epilogue == MNI_EPI_BIAS_RELU) v = fmaxf(v, 0.0f);
                        else if (g.epilogue == MNI_EPI_BIAS_GELU) v = gelu_tanh(v);
                        if (g.accumulate) v += *dst;
                    }
                    *dst = v;
                }
            }
        }
    }
}

int launch_gemm_mfma(const GemmLaunch &g, int amode, int bmode) {
    const int64_t blocks = (int64_t)g.tiles_m * g.tiles_n * g.batch * g.split_k;
    if (blocks <= 0) return MNI_OK;
    if (blocks > 0x7fffffffLL) return set_error(MNI_ERR_INVALID, "sgemm: too many tiles (%lld)", (long long)blocks);
    dim3 grid((unsigned)blocks), block(NTHREADS);
    hipStream_t s = ctx().stream;
#define MNI_LAUNCH(AM, BMO) hipLaunchKernelGGL((gemm_mfma_kernel<AM, BMO>), grid, block, 0, s, g)
    if (amode == 2 || bmode == 2) MNI_LAUNCH(2, 2);
    else if (amode == 0 && bmode == 0) MNI_LAUNCH(0, 0);
    else if (amode == 0 && bmode == 1) MNI_LAUNCH(0, 1);
    else if (amode == 1 && bmode == 0) MNI_LAUNCH(1, 0);
    else MNI_LAUNCH(1, 1);
#undef MNI_LAUNCH
    return check_launch("gemm_mfma_kernel");
}

int gemm_mfma_tile_m() { return BM; }
int gemm_mfma_tile_n() { return BN; }
int gemm_mfma_tile_k() { return BK; }

}  // namespace mni
