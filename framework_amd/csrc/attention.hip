// Softmax along one dim and the row kernels of attention built on the batched
// GEMM (scores = Q K^T, P = softmax(scale * scores [causal]), O = P V).
// Counterparts in the reference: ops/norm.rs:10-50, 96-123 (softmax and its
// backward) and ops/attention.rs:14-78, 143-202 (flash_attention and its
// backward), whose cuda arm (kernels/flash_attention.cu) walks the keys one by
// one per query row; here the two products run on the MFMA tile kernel and only
// the row-wise normalisation is left to these bandwidth kernels.
#include "common.h"

namespace mni {

static constexpr int ATT_TPB = 256;  // 4 wavefronts, one row each

static inline unsigned rows_grid(int64_t rows) { return (unsigned)((rows + 3) / 4); }

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// ---- softmax, contiguous lines (inner == 1): one wavefront per line -------------
__global__ void softmax_rows_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t rows, int64_t n) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *p = x + row * n;
    float *o = out + row * n;
    float mx = -INFINITY;
    for (int64_t j = lane; j < n; j += 64) mx = fmaxf(mx, p[j]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int64_t j = lane; j < n; j += 64) {
        const float e = expf(p[j] - mx);
        o[j] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    for (int64_t j = lane; j < n; j += 64) o[j] = o[j] / sum;
}
// lines of a few values: a thread per line (a wavefront per line leaves 60 lanes idle: 1 M lines of 4 took 250 us)
__global__ void softmax_short_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t rows, int n) {
    const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (row >= rows) return;
    const float *p = x + row * n;
    float *o = out + row * n;
    float v[16];
    float mx = -INFINITY;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        v[j] = j < n ? p[j] : -INFINITY;
        mx = fmaxf(mx, v[j]);
    }
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        v[j] = j < n ? expf(v[j] - mx) : 0.0f;
        sum += v[j];
    }
#pragma unroll
    for (int j = 0; j < 16; ++j)
        if (j < n) o[j] = v[j] / sum;
}
// long contiguous lines: a workgroup per line (a wavefront alone walks a vocabulary-sized line 786 steps at a
// time, three times over: 8 x 50304 took 624 us)
__global__ __launch_bounds__(1024) void softmax_lines_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t n, int vec) {
    __shared__ float red[32];
    float mx, sum;
    softmax_line_workgroup(out + (int64_t)blockIdx.x * n, x + (int64_t)blockIdx.x * n, n, vec != 0, red, mx, sum);
}
// lines of up to 1024 NV values in whole 16-byte pieces: a workgroup per line holds it in registers -- one read, one write
template <int NV>
__global__ __launch_bounds__(256) void softmax_lines_cached_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t n) {
    __shared__ float red[2][4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t n4 = n >> 2;
    const float4 *p = reinterpret_cast<const float4 *>(x + (int64_t)blockIdx.x * n);
    float4 *o = reinterpret_cast<float4 *>(out + (int64_t)blockIdx.x * n);
    float4 r[NV];
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t j = tid + 256 * i;
        r[i] = j < n4 ? p[j] : make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    }
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < NV; ++i) mx = fmaxf(fmaxf(mx, fmaxf(r[i].x, r[i].y)), fmaxf(r[i].z, r[i].w));
    mx = wave_max(mx);
    if (lane == 0) red[0][wave] = mx;
    __syncthreads();
    mx = fmaxf(fmaxf(red[0][0], red[0][1]), fmaxf(red[0][2], red[0][3]));
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        if (tid + 256 * i < n4) {
            r[i].x = expf(r[i].x - mx); r[i].y = expf(r[i].y - mx); r[i].z = expf(r[i].z - mx); r[i].w = expf(r[i].w - mx);
            sum += r[i].x; sum += r[i].y; sum += r[i].z; sum += r[i].w;
        }
    }
    sum = wave_sum(sum);
    if (lane == 0) red[1][wave] = sum;
    __syncthreads();
    sum = (red[1][0] + red[1][1]) + (red[1][2] + red[1][3]);
#pragma unroll
    for (int i = 0; i < NV; ++i) {
        const int64_t j = tid + 256 * i;
        if (j < n4) o[j] = make_float4(r[i].x / sum, r[i].y / sum, r[i].z / sum, r[i].w / sum);
    }
}
// lines with a stride (inner > 1): one thread per line, neighbours coalesce
__global__ void softmax_strided_kernel(float *__restrict__ out, const float *__restrict__ x, int64_t outer, int64_t n,
                                       int64_t inner) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t base = (idx / inner) * n * inner + idx % inner;
    float mx = -INFINITY;
    for (int64_t t = 0; t < n; ++t) mx = fmaxf(mx, x[base + t * inner]);
    float sum = 0.f;
    for (int64_t t = 0; t < n; ++t) {
        const float e = expf(x[base + t * inner] - mx);
        out[base + t * inner] = e;
        sum += e;
    }
    for (int64_t t = 0; t < n; ++t) out[base + t * inner] /= sum;
}
int k_softmax(float *out, const float *x, int64_t outer, int64_t n, int64_t inner) {
    if (outer * n * inner <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (inner == 1 && n <= 16 && outer >= 4096) {
        MNI_KERNEL_LAUNCH(softmax_short_kernel, dim3((unsigned)((outer + ATT_TPB - 1) / ATT_TPB)), dim3(ATT_TPB), 0, ctx().stream, out, x, outer, (int)n);
    } else if (inner == 1 && n >= 1024 && outer <= 0x7fffffffLL) {
        const int vec = n % 4 == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)x & 15) == 0;
        if (vec && n <= 2048) MNI_KERNEL_LAUNCH(softmax_lines_cached_kernel<2>, dim3((unsigned)outer), dim3(256), 0, ctx().stream, out, x, n);
        else if (vec && n <= 8192) MNI_KERNEL_LAUNCH(softmax_lines_cached_kernel<8>, dim3((unsigned)outer), dim3(256), 0, ctx().stream, out, x, n);
        else MNI_KERNEL_LAUNCH(softmax_lines_kernel, dim3((unsigned)outer), dim3(n <= 16384 ? 256 : 1024), 0, ctx().stream, out, x, n, vec);
    } else if (inner == 1)
        MNI_KERNEL_LAUNCH(softmax_rows_kernel, dim3(rows_grid(outer)), dim3(ATT_TPB), 0, ctx().stream, out, x, outer, n);
    else
        MNI_KERNEL_LAUNCH(softmax_strided_kernel, dim3((unsigned)((outer * inner + ATT_TPB - 1) / ATT_TPB)), dim3(ATT_TPB), 0,
                           ctx().stream, out, x, outer, n, inner);
    return check_launch("softmax");
}

// dx = sm * (g - sum(g * sm)) along the line
__global__ void softmax_bwd_rows_kernel(float *__restrict__ out, const float *__restrict__ sm, const float *__restrict__ g,
                                        int64_t rows, int64_t n) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    const float *s = sm + row * n, *gr = g + row * n;
    float dot = 0.f;
    for (int64_t j = lane; j < n; j += 64) dot += gr[j] * s[j];
    dot = wave_sum(dot);
    for (int64_t j = lane; j < n; j += 64) out[row * n + j] = s[j] * (gr[j] - dot);
}
// long lines: a workgroup per line (sums per thread, per wavefront, then in wavefront order)
__global__ __launch_bounds__(1024) void softmax_bwd_lines_kernel(float *__restrict__ out, const float *__restrict__ sm,
                                                                 const float *__restrict__ g, int64_t n) {
    __shared__ float red[16];
    const int tid = threadIdx.x, nt = blockDim.x, lane = tid & 63, wave = tid >> 6, nw = nt >> 6;
    const float *s = sm + (int64_t)blockIdx.x * n, *gr = g + (int64_t)blockIdx.x * n;
    float *o = out + (int64_t)blockIdx.x * n;
    float dot = 0.f;
    for (int64_t j = tid; j < n; j += nt) dot += gr[j] * s[j];
    dot = wave_sum(dot);
    if (lane == 0) red[wave] = dot;
    __syncthreads();
    dot = red[0];
    for (int w = 1; w < nw; ++w) dot += red[w];
    for (int64_t j = tid; j < n; j += nt) o[j] = s[j] * (gr[j] - dot);
}
__global__ void softmax_bwd_strided_kernel(float *__restrict__ out, const float *__restrict__ sm,
                                           const float *__restrict__ g, int64_t outer, int64_t n, int64_t inner) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= outer * inner) return;
    const int64_t base = (idx / inner) * n * inner + idx % inner;
    float dot = 0.f;
    for (int64_t t = 0; t < n; ++t) dot += g[base + t * inner] * sm[base + t * inner];
    for (int64_t t = 0; t < n; ++t) out[base + t * inner] = sm[base + t * inner] * (g[base + t * inner] - dot);
}
int k_softmax_backward(float *out, const float *sm, const float *g, int64_t outer, int64_t n, int64_t inner) {
    if (outer * n * inner <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (inner == 1 && n >= 2048 && outer <= 0x7fffffffLL)
        MNI_KERNEL_LAUNCH(softmax_bwd_lines_kernel, dim3((unsigned)outer), dim3(n <= 16384 ? 256 : 1024), 0, ctx().stream, out, sm, g, n);
    else if (inner == 1)
        MNI_KERNEL_LAUNCH(softmax_bwd_rows_kernel, dim3(rows_grid(outer)), dim3(ATT_TPB), 0, ctx().stream, out, sm, g, outer, n);
    else
        MNI_KERNEL_LAUNCH(softmax_bwd_strided_kernel, dim3((unsigned)((outer * inner + ATT_TPB - 1) / ATT_TPB)), dim3(ATT_TPB),
                           0, ctx().stream, out, sm, g, outer, n, inner);
    return check_launch("softmax_backward");
}

// ---- attention rows -----------------------------------------------------------------
// scores[rows = bh * s][s] holds q.k; in place: P = softmax over the allowed
// columns of scale * scores (col <= row % s when causal), 0 elsewhere, and
// lse[row] = max + ln(sum) (ops/attention.rs:33-60).  One wavefront per row;
// rows of up to 1024 columns stay in registers between the passes.
__global__ void attn_softmax_kernel(float *__restrict__ scores, float *__restrict__ lse, int64_t rows, int s, float scale,
                                    int causal) {
    constexpr int R = 16;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    float *p = scores + row * (int64_t)s;
    const int col_end = causal ? (int)(row % s) + 1 : s;
    if (s <= 64 * R) {
        float v[R];
        float mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int j = lane + 64 * i;
            v[i] = j < col_end ? p[j] * scale : -INFINITY;
            mx = fmaxf(mx, v[i]);
        }
        mx = wave_max(mx);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            v[i] = lane + 64 * i < col_end ? expf(v[i] - mx) : 0.f;
            sum += v[i];
        }
        sum = wave_sum(sum);
        const float inv = 1.0f / sum;
#pragma unroll
        for (int i = 0; i < R; ++i) {
            const int j = lane + 64 * i;
            if (j < s) p[j] = v[i] * inv;
        }
        if (lane == 0) lse[row] = mx + logf(sum);
        return;
    }
    float mx = -INFINITY;
    for (int j = lane; j < col_end; j += 64) mx = fmaxf(mx, p[j] * scale);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int j = lane; j < col_end; j += 64) sum += expf(p[j] * scale - mx);
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
    for (int j = lane; j < s; j += 64) p[j] = j < col_end ? expf(p[j] * scale - mx) * inv : 0.f;
    if (lane == 0) lse[row] = mx + logf(sum);
}
int k_attn_softmax(float *scores, float *lse, int64_t rows, int64_t s, float scale, int causal) {
    if (rows <= 0 || s <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(attn_softmax_kernel, dim3(rows_grid(rows)), dim3(ATT_TPB), 0, ctx().stream, scores, lse, rows, (int)s,
                       scale, causal);
    return check_launch("attn_softmax");
}

// ---- attention forward in one kernel --------------------------------------------------
// out = softmax(scale * q k^T [+ causal mask]) v and lse = max + ln(sum) per query
// (ops/attention.rs:14-78), for head dims 32, 64, 96, 128, without the s x s
// score matrix ever leaving the chip.  A workgroup owns 128 queries (32 per
// wavefront) and walks the keys 32 or 64 at a time with the running-maximum
// recurrence of the reference.  Both products run on v_mfma_f32_32x32x2_f32 and
// are taken transposed, which puts one query in every lane:
//   S^T = K Q^T   A = the key tile (LDS, [d/4][key] float4), B = the lane's own
//                 query row (registers); lane (query r, half h) receives the
//                 scores of keys 8(e/4) + 4h + e%4, e = 0..15, so the row
//                 maximum and sum are 15 in-lane steps and one exchange
//                 between the halves;
//   O^T += V^T P^T  the probabilities stay where they are: MFMA j of chunk c
//                 contracts keys 8c + 4h + j, which is exactly accumulator
//                 element 4c + j of S^T, so P^T is fed to the matrix pipe as
//                 operand B straight from the registers; A = V^T read from the
//                 value tile in LDS.  Rescaling the running output is one
//                 factor per lane.
typedef float att_f16 __attribute__((ext_vector_type(16)));

// Which block of which head a workgroup takes.  Under the causal mask the blocks of a head differ in
// work by a factor of up to their number, and the kernels below keep two workgroups on a CU, so what
// counts is the sum of the two that share one.  The hardware hands workgroup x and workgroup x + CUs to
// the same CU while the first two per CU are being placed.  With the blocks numbered from the heaviest
// (t = 0) and `pair` = CUs, the w = min(total - pair, pair) CUs that receive a second workgroup get
// blocks pair - w + x and pair + w - 1 - x: the lightest 2w of the first 2 pair blocks, folded so that
// heavy meets light, while the heaviest blocks run alone.  What is left after 2 pair workgroups goes on
// in falling order to the slots that free up.  pair is a huge value when only one workgroup fits a CU.
__device__ __forceinline__ void attn_item(int nblocks, int pair, int &rank, int64_t &bh) {
    const int total = (int)gridDim.x, heads = total / nblocks;
    int t = (int)blockIdx.x;
    if (total > pair && t - pair < pair) {
        const int w = min(total - pair, pair);
        if (t < w) t += pair - w;
        else if (t < pair) t -= w;
        else t = pair + w - 1 - (t - pair);
    }
    rank = t / heads;
    bh = t % heads;
}
static constexpr int AF_QUERIES = 128;
// SPLIT (with 64 keys per step): the workgroup owns 64 queries instead of 128 and its wavefronts pair up on
// them, one taking keys 0 .. 31 and the other keys 32 .. 63 of every tile; the two partial results (running
// maximum, sum and output) meet in LDS at the end.  Half the MFMAs per wavefront and step: for grids too
// small to fill the chip, where the time is that of the longest chain of steps (every head dim; 96 and 128
// then take 64-key tiles too, one workgroup per CU).
template <int DB, int NB, bool SPLIT>  // head dim = 32 * DB, keys per step = 32 * NB
__global__ __launch_bounds__(ATT_TPB, (SPLIT && DB > 2 ? 1 : 2)) void attn_fused_fwd_kernel(float *__restrict__ out, float *__restrict__ lse,
                                                                    const float *__restrict__ q, const float *__restrict__ k,
                                                                    const float *__restrict__ v, int s, int qblocks, int pair,
                                                                    float scale, int causal) {
    static_assert(!SPLIT || NB == 2, "the split form takes 64-key tiles");
    constexpr int D = 32 * DB, DQ = D / 4, KEYS = 32 * NB;
    constexpr int QB = SPLIT ? 64 : AF_QUERIES;  // queries per workgroup
    constexpr int NBW = SPLIT ? 1 : NB;          // blocks of 32 keys a wavefront takes out of a tile
    constexpr int KPITCH = KEYS + 1;  // float4 per d-quad slice (+1: the tile stores of consecutive quads spread over the banks)
    constexpr int VPITCH = D + 8;     // floats per key row (+8: the two lane halves, 4 keys apart, use different banks)
    constexpr int KSTAGE = DQ * KPITCH, VSTAGE = KEYS * VPITCH;
    constexpr int NLD = KEYS * DQ / ATT_TPB;  // float4 of each tile per thread (1 .. 4)
    __shared__ float4 kt[2 * KSTAGE];
    __shared__ __align__(16) float vt[2 * VSTAGE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int grp = SPLIT ? (wave & 1) : wave;      // which 32 queries of the workgroup
    const int koff = SPLIT ? 32 * (wave >> 1) : 0;  // first key of a tile this wavefront takes
    int rank;
    int64_t bh;
    attn_item(qblocks, pair, rank, bh);
    const int qb = qblocks - 1 - rank;  // late queries have the most keys to visit under the causal mask
    const int qi = qb * QB + grp * 32 + r;  // this lane's query
    const int ql = min(qi, s - 1);                   // (queries beyond the end compute on the last one and store nothing)
    const float *qrow = q + (bh * s + ql) * (int64_t)D;
    const float *kbase = k + bh * s * (int64_t)D, *vbase = v + bh * s * (int64_t)D;
    float4 qf[D / 8];  // the d quads 2c + h of the lane's query
#pragma unroll
    for (int c = 0; c < D / 8; ++c) qf[c] = *reinterpret_cast<const float4 *>(qrow + 4 * (2 * c + h));
    att_f16 oacc[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[b][e] = 0.f;
    float m = -INFINITY, l = 0.f;
    // keys this workgroup needs: all of them, or those up to its last query
    const int nkeys = causal ? min(s, (qb + 1) * QB) : s;
    const int nsteps = (nkeys + KEYS - 1) / KEYS;
    const int wave_first = qb * QB + grp * 32;  // first query of this wavefront
    const int wave_last = min(wave_first + 31, s - 1);   // and its last
    const float scale2 = scale * 1.4426950408889634f;    // scores in units of log2

    // Tiles travel global -> registers -> LDS; the registers are filled for step
    // i + 1 before step i is computed and parked in the other LDS stage after it,
    // so a request has a whole step to arrive and one barrier per step orders
    // everything.  Requests and stores are unconditional (the last step fetches
    // its own tile again into a stage nobody reads): a predicated refill would
    // be merged with the old register contents right behind the loads.
    float4 kreg[NLD], vreg[NLD];
    // where this thread's pieces of a tile come from and go to (the same for every step)
    int src_off[NLD], k_slot[NLD], v_slot[NLD], key_of[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int f = tid + ATT_TPB * i;
        key_of[i] = f / DQ;
        src_off[i] = 4 * (f % DQ);
        k_slot[i] = (f % DQ) * KPITCH + f / DQ;
        v_slot[i] = (f / DQ) * VPITCH + 4 * (f % DQ);
    }
#define MNI_AF_REQUEST(STEP)                                                                          \
    _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                                                 \
        const int64_t src = (int64_t)min((STEP) * KEYS + key_of[i], s - 1) * D + src_off[i];           \
        kreg[i] = *reinterpret_cast<const float4 *>(kbase + src);                                     \
        vreg[i] = *reinterpret_cast<const float4 *>(vbase + src);                                     \
    }
#define MNI_AF_PARK(STAGE)                                                                            \
    _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                                                 \
        kt[(STAGE) * KSTAGE + k_slot[i]] = kreg[i];                                                   \
        *reinterpret_cast<float4 *>(vt + (STAGE) * VSTAGE + v_slot[i]) = vreg[i];                     \
    }
    MNI_AF_REQUEST(0)
    MNI_AF_PARK(0)
    __syncthreads();
    for (int step = 0; step < nsteps; ++step) {
        const int k0 = step * KEYS;
        const int cur = step & 1;
        MNI_AF_REQUEST(min(step + 1, nsteps - 1))
        // a wavefront whose queries all come before this key tile has nothing to add (causal)
        if ((!causal || k0 + koff <= wave_last) && k0 + koff < s) {
            const float4 *ks = kt + cur * KSTAGE;
            const float *vs = vt + cur * VSTAGE;
            att_f16 sacc[NBW];
            bool live[NBW];  // under the causal mask the later 32 keys of a step may all lie past this wavefront
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb) {
                live[nb] = !causal || k0 + koff + 32 * nb <= wave_last;
#pragma unroll
                for (int e = 0; e < 16; ++e) sacc[nb][e] = 0.f;
                if (live[nb]) {
                    // key fragments are fetched from LDS one d chunk ahead of the MFMAs that use them
                    float4 ka = ks[h * KPITCH + koff + 32 * nb + r];
#pragma unroll
                    for (int c = 0; c < D / 8; ++c) {
                        float4 na = ka;
                        if (c + 1 < D / 8) na = ks[(2 * (c + 1) + h) * KPITCH + koff + 32 * nb + r];
                        sacc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.x, qf[c].x, sacc[nb], 0, 0, 0);
                        sacc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.y, qf[c].y, sacc[nb], 0, 0, 0);
                        sacc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.z, qf[c].z, sacc[nb], 0, 0, 0);
                        sacc[nb] = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.w, qf[c].w, sacc[nb], 0, 0, 0);
                        ka = na;
                    }
                }
            }
            // From here on in units of log2: p = 2^(x - max) is one v_exp_f32.  Only a tile that
            // reaches past the last key or across the diagonal of this wavefront needs the mask.
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
                for (int e = 0; e < 16; ++e) sacc[nb][e] *= scale2;
            if (k0 + KEYS > s || (causal && k0 + KEYS - 1 > wave_first)) {
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
                    for (int e = 0; e < 16; ++e) {
                        const int key = k0 + koff + 32 * nb + 8 * (e >> 2) + 4 * h + (e & 3);
                        if (!(key < s && (!causal || key <= ql))) sacc[nb][e] = -INFINITY;
                    }
            }
            float mx = m;
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
                for (int e = 0; e < 16; ++e) mx = fmaxf(mx, sacc[nb][e]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            // (key 0 is allowed for every query, so mx is finite from the first step on)
            const float alpha = __builtin_amdgcn_exp2f(m - mx);
            float psum = 0.f;
#pragma unroll
            for (int nb = 0; nb < NBW; ++nb)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    sacc[nb][e] = __builtin_amdgcn_exp2f(sacc[nb][e] - mx);
                    psum += sacc[nb][e];
                }
            psum += __shfl_xor(psum, 32, 64);
            l = l * alpha + psum;
            m = mx;
            // once the running maxima have settled nothing needs rescaling
            const bool rescale = __any(alpha != 1.0f) != 0;
#pragma unroll
            for (int b = 0; b < DB; ++b) {
                if (rescale) {
#pragma unroll
                    for (int e = 0; e < 16; ++e) oacc[b][e] *= alpha;
                }
#pragma unroll
                for (int nb = 0; nb < NBW; ++nb) {
                    if (!live[nb]) continue;
#pragma unroll
                    for (int c = 0; c < 4; ++c)
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            oacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vs[(koff + 32 * nb + 8 * c + 4 * h + j) * VPITCH + 32 * b + r],
                                                                           sacc[nb][4 * c + j], oacc[b], 0, 0, 0);
                }
            }
        }
        MNI_AF_PARK(cur ^ 1)
        __syncthreads();
    }
#undef MNI_AF_REQUEST
#undef MNI_AF_PARK
    if constexpr (SPLIT) {
        // The wavefronts of the second key half hand (output, maximum, sum) to their partners through the
        // tile memory, which the loop's last barrier has released: element x of lane l at [grp][x][l].
        constexpr int NX = 16 * DB + 2;
        static_assert(2 * NX * 64 * sizeof(float) <= sizeof(kt), "merge buffer must fit the key tiles");
        float *mb = reinterpret_cast<float *>(kt) + grp * NX * 64 + lane;
        if (koff != 0) {
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int e = 0; e < 16; ++e) mb[(16 * b + e) * 64] = oacc[b][e];
            mb[16 * DB * 64] = m;
            mb[(16 * DB + 1) * 64] = l;
        }
        __syncthreads();
        if (koff != 0) return;
        const float m1 = mb[16 * DB * 64], l1 = mb[(16 * DB + 1) * 64];
        const float mx = fmaxf(m, m1);  // m is finite: key 0 belongs to this half
        const float a0 = __builtin_amdgcn_exp2f(m - mx), a1 = __builtin_amdgcn_exp2f(m1 - mx);
        l = l * a0 + l1 * a1;
        m = mx;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) oacc[b][e] = oacc[b][e] * a0 + mb[(16 * b + e) * 64] * a1;
    }
    if (qi < s) {
        const float inv = 1.0f / l;
        float *orow = out + (bh * s + qi) * (int64_t)D;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)  // accumulator elements 4 g4 .. 4 g4 + 3 are d = 32 b + 8 g4 + 4 h + 0..3
                *reinterpret_cast<float4 *>(orow + 32 * b + 8 * g4 + 4 * h) =
                    make_float4(oacc[b][4 * g4] * inv, oacc[b][4 * g4 + 1] * inv, oacc[b][4 * g4 + 2] * inv, oacc[b][4 * g4 + 3] * inv);
        if (h == 0) lse[bh * s + qi] = m * 0.6931471805599453f + logf(l);  // back from log2 units
    }
}
// The distance in launch order between the two workgroups that share a CU (see attn_item): the number of
// CUs when at least two workgroups of `kernel` fit one, otherwise a value no grid reaches.
template <auto Kernel>
static int attn_pair() {
    static int fit = 0;  // per kernel instantiation; the answer does not change while the process lives
    if (fit == 0) {
        int n = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, Kernel, ATT_TPB, 0) != hipSuccess) (void)hipGetLastError();
        fit = n >= 1 ? n : 1;
    }
    const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
    return fit >= 2 ? cus : 0x7fffffff;
}

// Whether a grid of `blocks` 128-query (or 128-key) blocks runs in the split form: fewer than two blocks per CU
// at head dims 32 and 64, where two split workgroups fit a CU; at most one at 96 and 128, where one does.
static bool attn_split(int64_t d, int64_t blocks) {
    const int64_t cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
    return d > 64 ? blocks <= cus : blocks < 2 * cus;
}

bool attn_fused_supported(int64_t d) { return d == 32 || d == 64 || d == 96 || d == 128; }
int k_attn_fused_forward(float *out, float *lse, const float *q, const float *k, const float *v, int64_t bh, int64_t s, int64_t d,
                         float scale, int causal) {
    if (bh <= 0 || s <= 0) return MNI_OK;
    if (!attn_fused_supported(d)) return set_error(MNI_ERR_INVALID, "fused attention: head dim %lld is not 32, 64, 96 or 128", (long long)d);
    MNI_TRY(ensure_init());
    int64_t qblocks = (s + AF_QUERIES - 1) / AF_QUERIES;
    if (s > 0x7fffff00LL || bh * qblocks > 0x3fffffffLL) return set_error(MNI_ERR_INVALID, "fused attention: extent out of range");
    // Few blocks of 128 queries per CU: blocks of 64 with the keys of a 64-key tile split over two wavefronts,
    // so that the chain of steps each wavefront has to run is half as long.  Larger grids keep the CUs busy
    // either way and pay for reading every tile twice as often.
    const bool split = attn_split(d, bh * qblocks);
    if (split) qblocks = (s + 63) / 64;
    const dim3 grid((unsigned)(bh * qblocks)), block(ATT_TPB);
    hipStream_t st = ctx().stream;
#define MNI_AF(DBV, NBV, SPV)                                                                                               \
    MNI_KERNEL_LAUNCH((attn_fused_fwd_kernel<DBV, NBV, SPV>), grid, block, 0, st, out, lse, q, k, v, (int)s, (int)qblocks, \
                       attn_pair<attn_fused_fwd_kernel<DBV, NBV, SPV>>(), scale, causal)
    switch (d / 32) {
        // 64 keys per step while two workgroups still fit a CU's LDS, 32 beyond
        case 1: if (split) MNI_AF(1, 2, true); else MNI_AF(1, 2, false); break;
        case 2: if (split) MNI_AF(2, 2, true); else MNI_AF(2, 2, false); break;
        case 3: if (split) MNI_AF(3, 2, true); else MNI_AF(3, 1, false); break;
        default: if (split) MNI_AF(4, 2, true); else MNI_AF(4, 1, false); break;
    }
#undef MNI_AF
    return check_launch("attn_fused_forward");
}

// ---- attention backward, query side -----------------------------------------------------
// dq = dS k with dS = P (dP - di) scale, P = exp(scale q k^T - lse), dP = dO v^T
// (ops/attention.rs:143-202), for the head dims of the one-kernel forward and
// with the same layout: a workgroup owns 128 queries, one per lane, and walks
// the keys 32 at a time.  S^T = K Q^T and dP^T = V dO^T take the key / value
// tiles from LDS ([d/4][key] float4) and the lane's own q / dO rows from
// registers; lse and di are one scalar per lane; dS^T stays in the accumulator
// registers and is operand B of dQ^T += K^T dS^T, whose operand A is the key
// tile once more, read along d out of the same [d/4][key] quads.
// SPLIT: as in the forward, 64 queries per workgroup and 64 keys per step, of which a wavefront takes 32;
// the two partial dq of a query are plain sums and are added through the tile memory at the end.
// WIDE: 128 queries per workgroup as in the plain form, but 64 keys per step, both halves taken by every
// wavefront in turn: half as many tile hand-overs and barriers per key.
template <int DB, bool SPLIT, bool WIDE>
__global__ __launch_bounds__(ATT_TPB, (DB <= 2 ? 2 : 1)) void attn_fused_bwd_dq_kernel(float *__restrict__ dq, const float *__restrict__ q,
                                                                       const float *__restrict__ k, const float *__restrict__ v,
                                                                       const float *__restrict__ dout, const float *__restrict__ lse,
                                                                       const float *__restrict__ di, int s, int qblocks, int pair, float scale,
                                                                       int causal) {
    constexpr int D = 32 * DB, DQ = D / 4, KEYS = SPLIT || WIDE ? 64 : 32;
    constexpr int QB = SPLIT ? 64 : AF_QUERIES;
    constexpr int TPITCH = KEYS + 1;  // float4 per d-quad slice of a [d/4][key] tile
    constexpr int TSTAGE = DQ * TPITCH;
    constexpr int NLD = KEYS * DQ / ATT_TPB;  // float4 of each tile per thread (1 .. 4)
    __shared__ float4 kt[2 * TSTAGE];
    __shared__ float4 vt[2 * TSTAGE];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int grp = SPLIT ? (wave & 1) : wave;      // which 32 queries of the workgroup
    const int koff0 = SPLIT ? 32 * (wave >> 1) : 0;  // first key of a tile this wavefront takes
    int rank;
    int64_t bh;
    attn_item(qblocks, pair, rank, bh);
    const int qb = qblocks - 1 - rank;  // late query blocks have the most keys under the mask
    const int qi = qb * QB + grp * 32 + r;
    const int ql = min(qi, s - 1);
    const int64_t row = bh * s + ql;
    const float *kbase = k + bh * s * (int64_t)D, *vbase = v + bh * s * (int64_t)D;
    float4 qf[D / 8], gf[D / 8];  // the d quads 2c + h of the lane's q and dO rows
#pragma unroll
    for (int c = 0; c < D / 8; ++c) {
        qf[c] = *reinterpret_cast<const float4 *>(q + row * D + 4 * (2 * c + h));
        gf[c] = *reinterpret_cast<const float4 *>(dout + row * D + 4 * (2 * c + h));
    }
    const float lse2 = lse[row] * 1.4426950408889634f, dil = di[row];
    const float scale2 = scale * 1.4426950408889634f;
    att_f16 qacc[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int e = 0; e < 16; ++e) qacc[b][e] = 0.f;
    const int nkeys = causal ? min(s, (qb + 1) * QB) : s;
    const int nsteps = (nkeys + KEYS - 1) / KEYS;
    const int wave_first = qb * QB + grp * 32;
    const int wave_last = min(wave_first + 31, s - 1);

    float4 kreg[NLD], vreg[NLD];
    int src_off[NLD], t_slot[NLD], key_of[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int f = tid + ATT_TPB * i;
        key_of[i] = f / DQ;
        src_off[i] = 4 * (f % DQ);
        t_slot[i] = (f % DQ) * TPITCH + f / DQ;
    }
#define MNI_AB_REQUEST(STEP)                                                                          \
    _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                                                 \
        const int64_t src = (int64_t)min((STEP) * KEYS + key_of[i], s - 1) * D + src_off[i];           \
        kreg[i] = *reinterpret_cast<const float4 *>(kbase + src);                                     \
        vreg[i] = *reinterpret_cast<const float4 *>(vbase + src);                                     \
    }
#define MNI_AB_PARK(STAGE)                                                                            \
    _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                                                 \
        kt[(STAGE) * TSTAGE + t_slot[i]] = kreg[i];                                                   \
        vt[(STAGE) * TSTAGE + t_slot[i]] = vreg[i];                                                   \
    }
    MNI_AB_REQUEST(0)
    MNI_AB_PARK(0)
    __syncthreads();
    for (int step = 0; step < nsteps; ++step) {
        const int k0 = step * KEYS;
        const int cur = step & 1;
        MNI_AB_REQUEST(min(step + 1, nsteps - 1))
#pragma unroll 1
        for (int koff = koff0; koff < (WIDE ? 64 : koff0 + 32); koff += 32)
        if ((!causal || k0 + koff <= wave_last) && k0 + koff < s) {
            const float4 *ks = kt + cur * TSTAGE, *vs = vt + cur * TSTAGE;
            // the key tile read along d for dQ^T += K^T dS^T: element (key, d) is component d % 4 of quad [d / 4][key];
            // 4 lanes share a quad and the next 4 are a whole slice further, which keeps them on different banks
            const float *krow = reinterpret_cast<const float *>(ks) + ((r >> 2) * TPITCH + koff + 4 * h) * 4 + (r & 3);
            att_f16 sacc, pacc;
#pragma unroll
            for (int e = 0; e < 16; ++e) { sacc[e] = 0.f; pacc[e] = 0.f; }
#pragma unroll
            for (int c = 0; c < D / 8; ++c) {
                const float4 ka = ks[(2 * c + h) * TPITCH + koff + r], va = vs[(2 * c + h) * TPITCH + koff + r];
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.x, qf[c].x, sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x2f32(va.x, gf[c].x, pacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.y, qf[c].y, sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x2f32(va.y, gf[c].y, pacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.z, qf[c].z, sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x2f32(va.z, gf[c].z, pacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ka.w, qf[c].w, sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x2f32(va.w, gf[c].w, pacc, 0, 0, 0);
            }
            // dS^T = P^T (dP^T - di) scale, 0 where the mask (or the end of the keys) forbids
            const bool edge = k0 + koff + 32 > s || (causal && k0 + koff + 31 > wave_first);
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const float p = __builtin_amdgcn_exp2f(sacc[e] * scale2 - lse2);
                float ds = p * (pacc[e] - dil) * scale;
                if (edge) {
                    const int key = k0 + koff + 8 * (e >> 2) + 4 * h + (e & 3);
                    if (!(key < s && (!causal || key <= ql))) ds = 0.f;
                }
                sacc[e] = ds;
            }
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        qacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(krow[(8 * b * TPITCH + 8 * c + j) * 4], sacc[4 * c + j],
                                                                       qacc[b], 0, 0, 0);
        }
        MNI_AB_PARK(cur ^ 1)
        __syncthreads();
    }
#undef MNI_AB_REQUEST
#undef MNI_AB_PARK
    if constexpr (SPLIT) {
        // element x of lane l at [grp][x][l] of the tile memory, which the loop's last barrier has released
        static_assert(2 * 16 * DB * 64 * sizeof(float) <= sizeof(kt), "merge buffer must fit the key tiles");
        float *mb = reinterpret_cast<float *>(kt) + grp * 16 * DB * 64 + lane;
        if (koff0 != 0) {
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int e = 0; e < 16; ++e) mb[(16 * b + e) * 64] = qacc[b][e];
        }
        __syncthreads();
        if (koff0 != 0) return;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) qacc[b][e] += mb[(16 * b + e) * 64];
    }
    if (qi < s) {
        float *orow = dq + (bh * s + qi) * (int64_t)D;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4)
                *reinterpret_cast<float4 *>(orow + 32 * b + 8 * g4 + 4 * h) =
                    make_float4(qacc[b][4 * g4], qacc[b][4 * g4 + 1], qacc[b][4 * g4 + 2], qacc[b][4 * g4 + 3]);
    }
}
int k_attn_fused_backward_dq(float *dq, const float *q, const float *k, const float *v, const float *dout, const float *lse,
                             const float *di, int64_t bh, int64_t s, int64_t d, float scale, int causal) {
    if (bh <= 0 || s <= 0) return MNI_OK;
    if (!attn_fused_supported(d)) return set_error(MNI_ERR_INVALID, "fused attention: head dim %lld is not 32, 64, 96 or 128", (long long)d);
    MNI_TRY(ensure_init());
    int64_t qblocks = (s + AF_QUERIES - 1) / AF_QUERIES;
    if (s > 0x7fffff00LL || bh * qblocks > 0x3fffffffLL) return set_error(MNI_ERR_INVALID, "fused attention: extent out of range");
    const bool split = attn_split(d, bh * qblocks);
    if (split) qblocks = (s + 63) / 64;
    const dim3 grid((unsigned)(bh * qblocks)), block(ATT_TPB);
    hipStream_t st = ctx().stream;
#define MNI_AB(DBV, SPV)                                                                                                               \
    MNI_KERNEL_LAUNCH((attn_fused_bwd_dq_kernel<DBV, SPV, !SPV>), grid, block, 0, st, dq, q, k, v, dout, lse, di, (int)s, (int)qblocks, \
                       attn_pair<attn_fused_bwd_dq_kernel<DBV, SPV, !SPV>>(), scale, causal)
    switch (d / 32) {
        case 1: if (split) MNI_AB(1, true); else MNI_AB(1, false); break;
        case 2: if (split) MNI_AB(2, true); else MNI_AB(2, false); break;
        case 3: if (split) MNI_AB(3, true); else MNI_AB(3, false); break;
        default: if (split) MNI_AB(4, true); else MNI_AB(4, false); break;
    }
#undef MNI_AB
    return check_launch("attn_fused_backward_dq");
}

// ---- attention backward, key side ---------------------------------------------------------
// dv = P^T dO and dk = dS^T q with the roles swapped: a workgroup owns 128 keys,
// one per lane (its k and v rows in registers), and walks the queries 32 at a
// time.  S = Q K^T and dP = dO V^T take the query / dO tiles from LDS
// ([d/4][query] float4); lane (key r, half h) receives queries 8(e/4) + 4h + e%4,
// whose lse and di come from LDS four at a time.  P and dS stay in the
// accumulator registers as operand B of dV^T += dO^T P and dK^T += Q^T dS, whose
// operands A are the dO / query tiles once more, read along d out of the same quads.
// Under the causal mask a key block starts at its own first query.
// SPLIT: 64 keys per workgroup and 64 queries per step, of which a wavefront takes 32; the two partial dk and
// dv of a key are plain sums and are added through the tile memory at the end.
// WIDE: 128 keys per workgroup as in the plain form, but 64 queries per step, both halves taken by every
// wavefront in turn.
template <int DB, bool SPLIT, bool WIDE>
__global__ __launch_bounds__(ATT_TPB, (DB <= 2 ? 2 : 1)) void attn_fused_bwd_dkv_kernel(
    float *__restrict__ dk, float *__restrict__ dv, const float *__restrict__ q, const float *__restrict__ k,
    const float *__restrict__ v, const float *__restrict__ dout, const float *__restrict__ lse, const float *__restrict__ di, int s,
    int kblocks, int pair, float scale, int causal) {
    constexpr int D = 32 * DB, DQ = D / 4, QT = SPLIT || WIDE ? 64 : 32;
    constexpr int KB = SPLIT ? 64 : AF_QUERIES;  // keys per workgroup
    constexpr int TPITCH = QT + 1;
    constexpr int TSTAGE = DQ * TPITCH;
    constexpr int NLD = QT * DQ / ATT_TPB;
    __shared__ float4 qt[2 * TSTAGE];
    __shared__ float4 gt[2 * TSTAGE];
    __shared__ __align__(16) float lt[2 * QT];
    __shared__ __align__(16) float dt[2 * QT];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int r = lane & 31, h = lane >> 5;
    const int grp = SPLIT ? (wave & 1) : wave;      // which 32 keys of the workgroup
    const int qoff0 = SPLIT ? 32 * (wave >> 1) : 0;  // first query of a tile this wavefront takes
    int kb;  // early key blocks see the most queries under the mask
    int64_t bh;
    attn_item(kblocks, pair, kb, bh);
    const int kj = kb * KB + grp * 32 + r;  // this lane's key
    const int kl = min(kj, s - 1);
    const int64_t base = bh * s;
    const float *qbase = q + base * (int64_t)D, *gbase = dout + base * (int64_t)D;
    float4 kf[D / 8], vf[D / 8];  // the d quads 2c + h of the lane's k and v rows
#pragma unroll
    for (int c = 0; c < D / 8; ++c) {
        kf[c] = *reinterpret_cast<const float4 *>(k + (base + kl) * D + 4 * (2 * c + h));
        vf[c] = *reinterpret_cast<const float4 *>(v + (base + kl) * D + 4 * (2 * c + h));
    }
    const float scale2 = scale * 1.4426950408889634f;
    att_f16 kacc[DB], vacc[DB];
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int e = 0; e < 16; ++e) { kacc[b][e] = 0.f; vacc[b][e] = 0.f; }
    const int q_begin = causal ? kb * KB : 0;  // queries before the block's first key see none of its keys
    const int nsteps = (s - q_begin + QT - 1) / QT;    // >= 1: the block holds at least one key < s
    const int wave_first = kb * KB + grp * 32;  // first key of this wavefront

    float4 qreg[NLD], greg[NLD];
    float lreg, dreg;
    int src_off[NLD], t_slot[NLD], row_of[NLD];
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
        const int f = tid + ATT_TPB * i;
        row_of[i] = f / DQ;
        src_off[i] = 4 * (f % DQ);
        t_slot[i] = (f % DQ) * TPITCH + f / DQ;
    }
#define MNI_AK_REQUEST(STEP)                                                                          \
    _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                                                 \
        const int64_t src = (int64_t)min(q_begin + (STEP) * QT + row_of[i], s - 1) * D + src_off[i];   \
        qreg[i] = *reinterpret_cast<const float4 *>(qbase + src);                                     \
        greg[i] = *reinterpret_cast<const float4 *>(gbase + src);                                     \
    }                                                                                                 \
    lreg = lse[base + min(q_begin + (STEP) * QT + (tid & (QT - 1)), s - 1)] * 1.4426950408889634f;           \
    dreg = di[base + min(q_begin + (STEP) * QT + (tid & (QT - 1)), s - 1)];
#define MNI_AK_PARK(STAGE)                                                                            \
    _Pragma("unroll") for (int i = 0; i < NLD; ++i) {                                                 \
        qt[(STAGE) * TSTAGE + t_slot[i]] = qreg[i];                                                   \
        gt[(STAGE) * TSTAGE + t_slot[i]] = greg[i];                                                   \
    }                                                                                                 \
    if (tid < QT) { lt[(STAGE) * QT + tid] = lreg; dt[(STAGE) * QT + tid] = dreg; }
    MNI_AK_REQUEST(0)
    MNI_AK_PARK(0)
    __syncthreads();
    for (int step = 0; step < nsteps; ++step) {
        const int q0 = q_begin + step * QT;
        const int cur = step & 1;
        MNI_AK_REQUEST(min(step + 1, nsteps - 1))
        // a wavefront whose keys all come after this query tile receives nothing from it (causal)
#pragma unroll 1
        for (int qoff = qoff0; qoff < (WIDE ? 64 : qoff0 + 32); qoff += 32)
        if ((!causal || q0 + qoff + 31 >= wave_first) && q0 + qoff < s) {
            const float4 *qs = qt + cur * TSTAGE, *gs = gt + cur * TSTAGE;
            // the same tiles read along d for dV^T += dO^T P and dK^T += Q^T dS: element (query, d) is component d % 4 of
            // quad [d / 4][query]; 4 lanes share a quad and the next 4 are a whole slice further, which keeps them on
            // different banks
            const float *qrow = reinterpret_cast<const float *>(qs) + ((r >> 2) * TPITCH + qoff + 4 * h) * 4 + (r & 3);
            const float *grow = reinterpret_cast<const float *>(gs) + ((r >> 2) * TPITCH + qoff + 4 * h) * 4 + (r & 3);
            att_f16 sacc, pacc;
#pragma unroll
            for (int e = 0; e < 16; ++e) { sacc[e] = 0.f; pacc[e] = 0.f; }
#pragma unroll
            for (int c = 0; c < D / 8; ++c) {
                const float4 qa = qs[(2 * c + h) * TPITCH + qoff + r], ga = gs[(2 * c + h) * TPITCH + qoff + r];
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa.x, kf[c].x, sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ga.x, vf[c].x, pacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa.y, kf[c].y, sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ga.y, vf[c].y, pacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa.z, kf[c].z, sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ga.z, vf[c].z, pacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(qa.w, kf[c].w, sacc, 0, 0, 0);
                pacc = __builtin_amdgcn_mfma_f32_32x32x2f32(ga.w, vf[c].w, pacc, 0, 0, 0);
            }
            // P and dS for the queries 8 g + 4 h + 0..3 of accumulator elements 4 g .. 4 g + 3
            const bool edge = q0 + qoff + 32 > s || kj >= s || (causal && q0 + qoff < wave_first + 32);
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                const float4 l4 = *reinterpret_cast<const float4 *>(lt + cur * QT + qoff + 8 * g4 + 4 * h);
                const float4 d4 = *reinterpret_cast<const float4 *>(dt + cur * QT + qoff + 8 * g4 + 4 * h);
                const float ls[4] = {l4.x, l4.y, l4.z, l4.w}, dd[4] = {d4.x, d4.y, d4.z, d4.w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int e = 4 * g4 + j;
                    float p = __builtin_amdgcn_exp2f(sacc[e] * scale2 - ls[j]);
                    if (edge) {
                        const int query = q0 + qoff + 8 * g4 + 4 * h + j;
                        if (!(query < s && kj < s && (!causal || kj <= query))) p = 0.f;
                    }
                    sacc[e] = p;
                    pacc[e] = p * (pacc[e] - dd[j]) * scale;
                }
            }
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int at = (8 * b * TPITCH + 8 * c + j) * 4;
                        vacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(grow[at], sacc[4 * c + j], vacc[b], 0, 0, 0);
                        kacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(qrow[at], pacc[4 * c + j], kacc[b], 0, 0, 0);
                    }
        }
        MNI_AK_PARK(cur ^ 1)
        __syncthreads();
    }
#undef MNI_AK_REQUEST
#undef MNI_AK_PARK
    if constexpr (SPLIT) {
        // element x of lane l at [grp][x][l] of the tile memory, which the loop's last barrier has released
        static_assert(2 * 32 * DB * 64 * sizeof(float) <= sizeof(qt), "merge buffer must fit the query tiles");
        float *mb = reinterpret_cast<float *>(qt) + grp * 32 * DB * 64 + lane;
        if (qoff0 != 0) {
#pragma unroll
            for (int b = 0; b < DB; ++b)
#pragma unroll
                for (int e = 0; e < 16; ++e) {
                    mb[(32 * b + e) * 64] = kacc[b][e];
                    mb[(32 * b + 16 + e) * 64] = vacc[b][e];
                }
        }
        __syncthreads();
        if (qoff0 != 0) return;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                kacc[b][e] += mb[(32 * b + e) * 64];
                vacc[b][e] += mb[(32 * b + 16 + e) * 64];
            }
    }
    if (kj < s) {
        float *krow = dk + (base + kj) * (int64_t)D, *vrow = dv + (base + kj) * (int64_t)D;
#pragma unroll
        for (int b = 0; b < DB; ++b)
#pragma unroll
            for (int g4 = 0; g4 < 4; ++g4) {
                *reinterpret_cast<float4 *>(krow + 32 * b + 8 * g4 + 4 * h) =
                    make_float4(kacc[b][4 * g4], kacc[b][4 * g4 + 1], kacc[b][4 * g4 + 2], kacc[b][4 * g4 + 3]);
                *reinterpret_cast<float4 *>(vrow + 32 * b + 8 * g4 + 4 * h) =
                    make_float4(vacc[b][4 * g4], vacc[b][4 * g4 + 1], vacc[b][4 * g4 + 2], vacc[b][4 * g4 + 3]);
            }
    }
}
int k_attn_fused_backward_dkv(float *dk, float *dv, const float *q, const float *k, const float *v, const float *dout,
                              const float *lse, const float *di, int64_t bh, int64_t s, int64_t d, float scale, int causal) {
    if (bh <= 0 || s <= 0) return MNI_OK;
    if (!attn_fused_supported(d)) return set_error(MNI_ERR_INVALID, "fused attention: head dim %lld is not 32, 64, 96 or 128", (long long)d);
    MNI_TRY(ensure_init());
    int64_t kblocks = (s + AF_QUERIES - 1) / AF_QUERIES;
    if (s > 0x7fffff00LL || bh * kblocks > 0x3fffffffLL) return set_error(MNI_ERR_INVALID, "fused attention: extent out of range");
    const bool split = attn_split(d, bh * kblocks);
    if (split) kblocks = (s + 63) / 64;
    const dim3 grid((unsigned)(bh * kblocks)), block(ATT_TPB);
    hipStream_t st = ctx().stream;
#define MNI_AK(DBV, SPV)                                                                                                            \
    MNI_KERNEL_LAUNCH((attn_fused_bwd_dkv_kernel<DBV, SPV, !SPV>), grid, block, 0, st, dk, dv, q, k, v, dout, lse, di, (int)s, (int)kblocks, \
                       attn_pair<attn_fused_bwd_dkv_kernel<DBV, SPV, !SPV>>(), scale, causal)
    switch (d / 32) {
        case 1: if (split) MNI_AK(1, true); else MNI_AK(1, false); break;
        case 2: if (split) MNI_AK(2, true); else MNI_AK(2, false); break;
        case 3: if (split) MNI_AK(3, true); else MNI_AK(3, false); break;
        default: if (split) MNI_AK(4, true); else MNI_AK(4, false); break;
    }
#undef MNI_AK
    return check_launch("attn_fused_backward_dkv");
}

// di[row] = sum_d a[row][d] * b[row][d] (ops/attention.rs:167-170)
__global__ void rowdot_kernel(float *__restrict__ out, const float *__restrict__ a, const float *__restrict__ b, int64_t rows,
                              int64_t d) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= rows) return;
    float t = 0.f;
    for (int64_t j = lane; j < d; j += 64) t += a[row * d + j] * b[row * d + j];
    t = wave_sum(t);
    if (lane == 0) out[row] = t;
}
int k_rowdot(float *out, const float *a, const float *b, int64_t rows, int64_t d) {
    if (rows <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    MNI_KERNEL_LAUNCH(rowdot_kernel, dim3(rows_grid(rows)), dim3(ATT_TPB), 0, ctx().stream, out, a, b, rows, d);
    return check_launch("rowdot");
}

// In place over scores (q.k) and dp (dO.v), both [rows][s]:
//   P  = exp(scale * scores - lse[row]) on the allowed columns, 0 elsewhere
//   dS = P * (dp - di[row]) * scale                     (ops/attention.rs:172-187)
__global__ void attn_bwd_kernel(float *__restrict__ scores, float *__restrict__ dp, const float *__restrict__ lse,
                                const float *__restrict__ di, int64_t rows, int s, float scale, int causal) {
    const int64_t n = rows * (int64_t)s;
    int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t step = (int64_t)gridDim.x * blockDim.x;
    for (; idx < n; idx += step) {
        const int64_t row = idx / s;
        const int col = (int)(idx - row * s);
        const bool on = !causal || col <= (int)(row % s);
        const float p = on ? expf(scores[idx] * scale - lse[row]) : 0.f;
        scores[idx] = p;
        dp[idx] = p * (dp[idx] - di[row]) * scale;
    }
}
int k_attn_backward(float *scores, float *dp, const float *lse, const float *di, int64_t rows, int64_t s, float scale,
                    int causal) {
    const int64_t n = rows * s;
    if (n <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    int64_t blocks = (n + ATT_TPB * 4 - 1) / (ATT_TPB * 4);
    if (blocks > 65536) blocks = 65536;
    MNI_KERNEL_LAUNCH(attn_bwd_kernel, dim3((unsigned)blocks), dim3(ATT_TPB), 0, ctx().stream, scores, dp, lse, di, rows,
                       (int)s, scale, causal);
    return check_launch("attn_backward");
}


// ---- device-resident KV cache -----------------------------------------------------------
// Counterpart of ops/kv_cache.rs, whose cache lives in host memory and whose
// decode loops over the history on the CPU (its cuda arm only quantises on the
// device).  Storage here is [bh, max_seq, d] in HBM, fp32 or int8 with one f32
// scale per row.

// append, fp32: row r of k / v goes to position pos of its head (:159-167)
__global__ void kv_append_f32_kernel(float *__restrict__ kc, float *__restrict__ vc, const float *__restrict__ k,
                                     const float *__restrict__ v, int64_t n, int64_t d, int64_t max_seq, int64_t pos) {
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= n) return;
    const int64_t row = idx / d, dd = idx - row * d;
    const int64_t dst = (row * max_seq + pos) * d + dd;
    kc[dst] = k[idx];
    vc[dst] = v[idx];
}
// append, int8: quantize_row_i8 (:357-370) -- scale = max(max|x| / 127, 1e-8),
// q = clamp(round(x * (1 / scale)), -127, 127), round half away from zero.
// One wavefront per (row, k or v).
__global__ void kv_append_i8_kernel(signed char *__restrict__ kc, signed char *__restrict__ vc, float *__restrict__ ks,
                                    float *__restrict__ vs, const float *__restrict__ k, const float *__restrict__ v,
                                    int64_t bh, int64_t d, int64_t max_seq, int64_t pos) {
    const int lane = threadIdx.x & 63;
    const int64_t job = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (job >= 2 * bh) return;
    const int64_t row = job >> 1;
    const bool is_v = job & 1;
    const float *src = (is_v ? v : k) + row * d;
    signed char *dst = (is_v ? vc : kc) + (row * max_seq + pos) * d;
    float mx = 0.f;
    for (int64_t j = lane; j < d; j += 64) mx = fmaxf(mx, fabsf(src[j]));
    mx = wave_max(mx);
    float scale = mx / 127.0f;
    if (!(scale > 1e-8f)) scale = 1e-8f;
    const float inv = 1.0f / scale;
    for (int64_t j = lane; j < d; j += 64) {
        float q = roundf(src[j] * inv);
        q = q < -127.0f ? -127.0f : q > 127.0f ? 127.0f : q;
        dst[j] = (signed char)q;
    }
    if (lane == 0) (is_v ? vs : ks)[row * max_seq + pos] = scale;
}
int k_kv_append(void *kc, void *vc, float *ks, float *vs, const float *k, const float *v, int64_t bh, int64_t d,
                int64_t max_seq, int64_t pos, int quantized) {
    if (bh * d <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (quantized)
        MNI_KERNEL_LAUNCH(kv_append_i8_kernel, dim3(rows_grid(2 * bh)), dim3(ATT_TPB), 0, ctx().stream, (signed char *)kc,
                           (signed char *)vc, ks, vs, k, v, bh, d, max_seq, pos);
    else
        MNI_KERNEL_LAUNCH(kv_append_f32_kernel, dim3((unsigned)((bh * d + ATT_TPB - 1) / ATT_TPB)), dim3(ATT_TPB), 0,
                           ctx().stream, (float *)kc, (float *)vc, k, v, bh * d, d, max_seq, pos);
    return check_launch("kv_append");
}

// decode (:259-287): attention of one query row per head over positions
// [0, len).  grid = (bh, splits): a workgroup takes a chunk of the history --
// one thread per key for the scores (the query sits in LDS), block-wide max and
// sum, then threads own output columns for the weighted sum of the values.  With
// more than one split the chunks leave (acc, max, sum) behind and
// kv_combine_kernel merges them (the usual log-sum-exp merge); the merge order is
// fixed, so results do not depend on scheduling.
struct KvDecode {
    const void *kc, *vc;
    const float *ks, *vs, *q;
    float *out, *part;  // part: [bh][splits][d + 2]
    int64_t d, max_seq;
    int len, splits, chunk;
    float scale;
};
static constexpr int KV_CHUNK_MAX = 2048;

__device__ __forceinline__ float block_reduce(float v, float *red, bool is_max) {
    v = is_max ? wave_max(v) : wave_sum(v);
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[w] = v;
    __syncthreads();
    float r = red[0];
    for (int i = 1; i < ATT_TPB / 64; ++i) r = is_max ? fmaxf(r, red[i]) : r + red[i];
    return r;
}

template <bool Q8>
__global__ __launch_bounds__(ATT_TPB) void kv_decode_kernel(const KvDecode a) {
    extern __shared__ float sm[];
    float *qs = sm;                 // [d]
    float *sc = sm + a.d;           // [chunk]
    float *red = sc + a.chunk;      // [ATT_TPB]
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x;
    const int sp = blockIdx.y;
    const int t0 = sp * a.chunk;
    const int n = min(a.len, t0 + a.chunk) - t0;
    const int64_t d = a.d;
    for (int64_t dd = tid; dd < d; dd += ATT_TPB) qs[dd] = a.q[row * d + dd];
    __syncthreads();
    // scores
    for (int i = tid; i < n; i += ATT_TPB) {
        const int64_t pos = row * a.max_seq + t0 + i;
        float dot = 0.f;
        if (Q8) {
            const signed char *kp = (const signed char *)a.kc + pos * d;
            const float s = a.ks[pos];
            for (int64_t dd = 0; dd < d; ++dd) dot += qs[dd] * ((float)kp[dd] * s);
        } else {
            const float *kp = (const float *)a.kc + pos * d;
            for (int64_t dd = 0; dd < d; ++dd) dot += qs[dd] * kp[dd];
        }
        sc[i] = dot * a.scale;
    }
    __syncthreads();
    float m = -INFINITY;
    for (int i = tid; i < n; i += ATT_TPB) m = fmaxf(m, sc[i]);
    m = block_reduce(m, red, true);
    float l = 0.f;
    for (int i = tid; i < n; i += ATT_TPB) {
        const float w = expf(sc[i] - m);
        sc[i] = w;
        l += w;
    }
    l = block_reduce(l, red, false);
    __syncthreads();
    // weighted sum of the values: threads own columns, groups split the keys
    const int lanes = d <= ATT_TPB ? (int)d : ATT_TPB;
    const int groups = d <= ATT_TPB ? ATT_TPB / (int)d : 1;
    float *pout = a.part + ((int64_t)row * a.splits + sp) * (d + 2);
    for (int64_t base = 0; base < d; base += lanes) {
        const int col = tid % lanes, grp = tid / lanes;
        const int64_t dd = base + col;
        float acc = 0.f;
        if (grp < groups && dd < d) {
            for (int i = grp; i < n; i += groups) {
                const int64_t pos = row * a.max_seq + t0 + i;
                const float vv = Q8 ? (float)((const signed char *)a.vc)[pos * d + dd] * a.vs[pos]
                                    : ((const float *)a.vc)[pos * d + dd];
                acc += sc[i] * vv;
            }
        }
        __syncthreads();
        red[tid] = acc;
        __syncthreads();
        if (tid < lanes && base + tid < d) {
            float s = 0.f;
            for (int g = 0; g < groups; ++g) s += red[g * lanes + tid];
            if (a.splits == 1) a.out[row * d + base + tid] = l > 0.f ? s * (1.0f / l) : 0.f;
            else pout[base + tid] = s;
        }
    }
    if (a.splits > 1 && tid == 0) { pout[d] = m; pout[d + 1] = l; }
}
// The same decode for head dims up to 256 (fp32, multiples of 4) or up to 1024
// (int8, multiples of 16): every row of the cache is read as 16-byte pieces by
// LPR neighbouring lanes -- 4 fp32 or 16 int8 values per lane -- so loads are
// coalesced; a dot product is finished with log2(LPR) butterfly steps, and the
// value pass keeps those 4 / 16 columns per lane.
template <bool Q8, int LPR>
__global__ __launch_bounds__(ATT_TPB) void kv_decode_vec_kernel(const KvDecode a) {
    constexpr int E = Q8 ? 16 : 4;         // elements per lane
    constexpr int KV_UNROLL = 4;           // cache rows in flight per lane (8 measured the same for int8, slower for fp32)
    constexpr int RPP = 64 / LPR;          // rows per wavefront pass
    constexpr int GROUPS = ATT_TPB / LPR;  // key groups in the value pass
    extern __shared__ float sm[];
    float *sc = sm;                         // [chunk]
    float *red = sm + a.chunk;              // [ATT_TPB]
    float *redv = red + ATT_TPB;            // [ATT_TPB][E]
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l = lane % LPR, sub = lane / LPR;
    const int64_t row = blockIdx.x;
    const int sp = blockIdx.y;
    const int t0 = sp * a.chunk;
    const int n = min(a.len, t0 + a.chunk) - t0;
    const int pieces = (int)(a.d / E);
    const int64_t base = row * a.max_seq + t0;
    // A 16-byte piece of a cache row is requested as it is stored (and, for
    // int8, the row's scale); it is widened to floats only where it is used, so
    // that the requests of a trip are all issued before the first wait.
    auto request = [&](const void *cache, const float *scales, int64_t pos, int piece, int4 &w, float &s) {
        if (Q8) {
            w = reinterpret_cast<const int4 *>(reinterpret_cast<const signed char *>(cache) + pos * a.d)[piece];
            s = scales[pos];
        } else {
            w = reinterpret_cast<const int4 *>(reinterpret_cast<const float *>(cache) + pos * a.d)[piece];
            s = 1.0f;
        }
    };
    auto widen = [&](const int4 &w, float s, float (&v)[E]) {
        const int ws[4] = {w.x, w.y, w.z, w.w};
        if (Q8) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int b8 = 0; b8 < 4; ++b8) v[4 * j + b8] = (float)(signed char)((ws[j] >> (8 * b8)) & 0xff) * s;
        } else {
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] = __int_as_float(ws[j]);
        }
    };
    float qv[E];
#pragma unroll
    for (int e = 0; e < E; ++e) qv[e] = l < pieces ? a.q[row * a.d + l * E + e] : 0.f;
    // scores: KV_UNROLL rows of the cache are requested before the first is used
    // (one 16-byte load per lane in flight does not cover the memory latency)
    constexpr int ROWS_PER_TRIP = (ATT_TPB / 64) * RPP;
    for (int i0 = wave * RPP; i0 < n; i0 += ROWS_PER_TRIP * KV_UNROLL) {
        int4 kw[KV_UNROLL];
        float ksc[KV_UNROLL];
#pragma unroll
        for (int u = 0; u < KV_UNROLL; ++u) {
            const int i = i0 + u * ROWS_PER_TRIP + sub;
            kw[u] = make_int4(0, 0, 0, 0);
            ksc[u] = 0.f;
            if (i < n && l < pieces) request(a.kc, a.ks, base + i, l, kw[u], ksc[u]);
        }
#pragma unroll
        for (int u = 0; u < KV_UNROLL; ++u) {
            const int i = i0 + u * ROWS_PER_TRIP + sub;
            float part = 0.f;
            if (i < n && l < pieces) {
                float kv[E];
                widen(kw[u], ksc[u], kv);
#pragma unroll
                for (int e = 0; e < E; ++e) part += qv[e] * kv[e];
            }
#pragma unroll
            for (int off = LPR / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, 64);
            if (i < n && l == 0) sc[i] = part * a.scale;
        }
    }
    __syncthreads();
    float m = -INFINITY;
    for (int i = tid; i < n; i += ATT_TPB) m = fmaxf(m, sc[i]);
    m = block_reduce(m, red, true);
    float lsum = 0.f;
    for (int i = tid; i < n; i += ATT_TPB) {
        const float w = expf(sc[i] - m);
        sc[i] = w;
        lsum += w;
    }
    lsum = block_reduce(lsum, red, false);
    __syncthreads();
    // values: lane lv of key group grp accumulates columns E * lv .. E * lv + E - 1
    const int lv = tid % LPR, grp = tid / LPR;
    float acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = 0.f;
    if (lv < pieces) {
        for (int i0 = grp; i0 < n; i0 += GROUPS * KV_UNROLL) {
            int4 vw[KV_UNROLL];
            float vsc[KV_UNROLL];
#pragma unroll
            for (int u = 0; u < KV_UNROLL; ++u) {
                vw[u] = make_int4(0, 0, 0, 0);
                vsc[u] = 0.f;
                if (i0 + u * GROUPS < n) request(a.vc, a.vs, base + i0 + u * GROUPS, lv, vw[u], vsc[u]);
            }
#pragma unroll
            for (int u = 0; u < KV_UNROLL; ++u) {
                const int i = i0 + u * GROUPS;
                if (i < n) {
                    const float w = sc[i];
                    float vv[E];
                    widen(vw[u], vsc[u], vv);
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[e] += w * vv[e];
                }
            }
        }
    }
#pragma unroll
    for (int e = 0; e < E; ++e) redv[e * ATT_TPB + tid] = acc[e];
    __syncthreads();
    float *pout = a.part + ((int64_t)row * a.splits + sp) * (a.d + 2);
    const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;
    // one thread per output column: column c = E * piece + e lives at redv[e][g * LPR + piece]
    for (int c = tid; c < (int)a.d; c += ATT_TPB) {
        const int piece = c / E, e = c % E;
        float s1 = 0.f;
        for (int g = 0; g < GROUPS; ++g) s1 += redv[e * ATT_TPB + g * LPR + piece];
        if (a.splits == 1) a.out[row * a.d + c] = s1 * inv;
        else pout[c] = s1;
    }
    if (a.splits > 1 && tid == 0) { pout[a.d] = m; pout[a.d + 1] = lsum; }
}
template <bool Q8>
static bool launch_kv_decode_vec(const KvDecode &a, dim3 grid, size_t lds) {
    const int pieces = (int)(a.d / (Q8 ? 16 : 4));
    hipStream_t st = ctx().stream;
#define MNI_KVV(L) MNI_KERNEL_LAUNCH((kv_decode_vec_kernel<Q8, L>), grid, dim3(ATT_TPB), lds, st, a)
    if (pieces <= 1) MNI_KVV(1);
    else if (pieces <= 2) MNI_KVV(2);
    else if (pieces <= 4) MNI_KVV(4);
    else if (pieces <= 8) MNI_KVV(8);
    else if (pieces <= 16) MNI_KVV(16);
    else if (pieces <= 32) MNI_KVV(32);
    else if (pieces <= 64) MNI_KVV(64);
    else return false;
#undef MNI_KVV
    return true;
}

__global__ void kv_combine_kernel(float *__restrict__ out, const float *__restrict__ part, int64_t d, int splits) {
    const int64_t row = blockIdx.x;
    const float *p = part + row * splits * (d + 2);
    float m = -INFINITY;
    for (int s = 0; s < splits; ++s) m = fmaxf(m, p[s * (d + 2) + d]);
    float l = 0.f;
    for (int s = 0; s < splits; ++s) l += p[s * (d + 2) + d + 1] * expf(p[s * (d + 2) + d] - m);
    const float inv = l > 0.f ? 1.0f / l : 0.f;
    for (int64_t dd = threadIdx.x; dd < d; dd += blockDim.x) {
        float acc = 0.f;
        for (int s = 0; s < splits; ++s) acc += p[s * (d + 2) + dd] * expf(p[s * (d + 2) + d] - m);
        out[row * d + dd] = acc * inv;
    }
}
int k_kv_decode(float *out, const void *kc, const void *vc, const float *ks, const float *vs, const float *q, int64_t bh,
                int64_t d, int64_t max_seq, int64_t len, float scale, int quantized) {
    if (bh <= 0 || d <= 0) return MNI_OK;
    MNI_TRY(ensure_init());
    if (len <= 0) return k_fill(out, 0.0f, bh * d);
    if (d > 4096) return set_error(MNI_ERR_INVALID, "kv cache decode: head_dim %lld above 4096", (long long)d);
    if (bh > 0x7fffffff || len > 0x7ffffff0) return set_error(MNI_ERR_INVALID, "kv cache decode: extent out of range");
    // enough workgroups to occupy the device, chunks of at most KV_CHUNK_MAX keys
    const int cus = ctx().compute_units > 0 ? ctx().compute_units : 256;
    int64_t splits = (4LL * cus + bh - 1) / bh;
    const int64_t max_by_len = (len + 127) / 128;
    if (splits > max_by_len) splits = max_by_len;
    const int64_t min_by_chunk = (len + KV_CHUNK_MAX - 1) / KV_CHUNK_MAX;
    if (splits < min_by_chunk) splits = min_by_chunk;
    if (splits < 1) splits = 1;
    int64_t chunk = (len + splits - 1) / splits;
    chunk = (chunk + 63) / 64 * 64;
    splits = (len + chunk - 1) / chunk;
    if (splits > 65535) return set_error(MNI_ERR_INVALID, "kv cache decode: history of %lld positions is too long", (long long)len);
    KvDecode a;
    a.kc = kc; a.vc = vc; a.ks = ks; a.vs = vs; a.q = q; a.out = out; a.part = nullptr;
    a.d = d; a.max_seq = max_seq; a.len = (int)len; a.splits = (int)splits; a.chunk = (int)chunk; a.scale = scale;
    void *part = nullptr;
    if (splits > 1) {
        MNI_TRY(dev_alloc(&part, (size_t)(bh * splits * (d + 2)) * sizeof(float)));
        a.part = (float *)part;
    } else {
        a.part = out;  // not written when splits == 1; keeps the pointer arithmetic in bounds
    }
    const dim3 grid((unsigned)bh, (unsigned)splits);
    // 16-byte pieces of a row: 4 fp32 or 16 int8 values (rows are then 16-byte aligned in the cache)
    const int per_lane = quantized ? 16 : 4;
    bool launched = false;
    if (d % per_lane == 0 && d / per_lane <= 64) {
        const size_t ldsv = (size_t)(chunk + ATT_TPB + per_lane * ATT_TPB) * sizeof(float);
        launched = quantized ? launch_kv_decode_vec<true>(a, grid, ldsv) : launch_kv_decode_vec<false>(a, grid, ldsv);
    }
    if (!launched) {
        const size_t lds = (size_t)(d + chunk + ATT_TPB) * sizeof(float);
        if (quantized) MNI_KERNEL_LAUNCH((kv_decode_kernel<true>), grid, dim3(ATT_TPB), lds, ctx().stream, a);
        else MNI_KERNEL_LAUNCH((kv_decode_kernel<false>), grid, dim3(ATT_TPB), lds, ctx().stream, a);
    }
    int rc = check_launch("kv_decode");
    if (rc == MNI_OK && splits > 1) {
        MNI_KERNEL_LAUNCH(kv_combine_kernel, dim3((unsigned)bh), dim3(ATT_TPB), 0, ctx().stream, out, (const float *)part, d,
                           (int)splits);
        rc = check_launch("kv_combine");
    }
    if (part) dev_free(part);
    return rc;
}

}  // namespace mni
