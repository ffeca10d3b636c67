// Skinny (GEMV-shaped) fp32 products for gfx950: a few rows of X against a
// large W.  These are bound by streaming W once from HBM, so they use plain
// FMAs, 16-byte loads with many loads in flight per lane, and wavefront / LDS
// reductions -- no MFMA.  The reference has no such special case: its cuda arm
// sends every shape to cuBLAS (src/native/src/ops/matmul.rs:150-189).
#include "common.h"
#include "gemm_internal.h"

namespace mni {

static constexpr int SK_THREADS = 256;   // skinny_cols: 4 wavefronts per workgroup
static constexpr int SK_WAVES = SK_THREADS / 64;
static constexpr int SK_COLS = 256;      // columns per workgroup: 64 lanes x float4
static constexpr int SK_UNROLL = 16;     // W rows in flight per lane
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float sk_gelu(float x) {
    const float s = 0.7978845608028654f;
    return 0.5f * x * (1.0f + tanhf(s * (x + 0.044715f * x * x * x)));
}

__device__ __forceinline__ float sk_epilogue(float v, float bias, int epilogue) {
    v += bias;
    if (epilogue == MNI_EPI_BIAS_RELU) v = fmaxf(v, 0.0f);
    else if (epilogue == MNI_EPI_BIAS_GELU) v = sk_gelu(v);
    return v;
}

// ---- W contiguous along columns ---------------------------------------------
// Work item = (column group of 256, K slice, batch), 256 threads = 4 wavefronts.
// A wavefront reads whole 1 KiB pieces of W rows (every lane one 16-byte load
// per row, SK_UNROLL rows in flight), which is the access pattern that streams
// HBM best; the X values of a row are the same for all lanes, so they are
// fetched with wave-uniform (scalar) loads.  The 4 wavefronts interleave groups
// of SK_UNROLL rows and are summed through LDS in wave order.  K is sliced
// across workgroups until about 4 workgroups per CU exist; each slice leaves a
// partial [slice][batch][rows][cols] and the slices are summed in a fixed
// order, so the result does not depend on scheduling.
//
// Who sums the slices:
//  * FUSED = false: a second launch (skinny_reduce_kernel).
//  * FUSED = true: the same launch.  All slices of a (batch, column group) unit
//    are given to workgroups of ONE XCD (1-D grid, workgroup b runs on XCD
//    b % xcds -- confirmed by a probe when the library starts), so the partials
//    never have to leave that XCD's L2.  A workgroup stores its partial, waits
//    for the stores to be acknowledged, then sets its own arrival flag to this
//    launch's epoch (a plain store to a private address).  The workgroups
//    holding the last R = min(rows, slices) slices of a unit then act as
//    reducers, one output row each: they poll the unit's flags with loads that
//    skip the CU's L1, read the row's partials from L2 and apply the epilogue.
//    Reducers wait for every slice of their unit, the later reducers' own
//    included, and a workgroup that waits keeps its place on its CU: were there
//    more reducers on an XCD than workgroups fit on it together, the first
//    ones could fill it and wait for slices that are never dispatched.  The
//    host therefore limits the reducers of a unit (max_reducers; each then
//    takes every max_reducers-th row) so that all reducers of an XCD fit on it
//    at once (skinny_cols_fused_occupancy), and takes the two-launch form when
//    not even one per unit does; the non-reducers ahead of them in the grid
//    never wait and make room as they finish.  The poll is bounded
//    all the same, and a reducer that gives up writes NaN and raises the
//    device status word.
//    Measured on MI355X for x[4,4096] W[4096,4096]: 12.2 us against 15.8 us for
//    two launches.  What does not work here: one arrival counter per unit
//    (returning atomics on one address serialise at ~145 ns each in L2: +9 us
//    for 64 slices), device-scope fences (L2 write-back per workgroup) and
//    float atomics.
static constexpr int SK_SPIN_LIMIT = 1 << 18;

__device__ __forceinline__ unsigned sk_load_flag(const unsigned *p) {
    // sc1: served by the XCD's L2, never by the CU's L1 (a plain load would
    // keep hitting the stale L1 line)
    unsigned v;
    asm volatile("global_load_dword %0, %1, off sc1\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
    return v;
}

// TAIL = false promises that every slice is a whole number of SK_UNROLL-row
// groups (K % SK_UNROLL == 0), which removes the guarded path and its address
// arithmetic from the kernel; this kernel lives for a few microseconds, so the
// length of its prologue shows.
template <int MR, bool XC, bool FUSED, bool TAIL, bool LEAN, bool PLAIN = false>
__global__ __launch_bounds__(SK_THREADS) void skinny_cols_kernel(const SkinnyLaunch s) {
    constexpr int U = SK_UNROLL;
    // LEAN (the decode shape): one batch, exactly MR rows, whole 256-column
    // groups, row-major output, a bias (if any) along the columns -- known at
    // compile time, so the general case's address arithmetic and guards drop
    // out of a kernel whose whole life is a few microseconds.  (The epilogue
    // stays a run-time choice: it is applied once per output at the very end.)  Instantiated for every row count from
    // 1 to 8 (and 16): with the count a run-time value below MR the guards come
    // back and cost 0.4 (4 rows) to 0.9 us (8 rows); with the count rounded up
    // to 4 or 8, x[1,4096] W[4096,4096] took 12.8 us against 11.7, 5 rows 15.7
    // against 13.4 (MI355X, W in the Infinity Cache).
    static_assert(!LEAN || (XC && FUSED && !TAIL), "LEAN implies XC, FUSED, !TAIL");
    const int rows = LEAN ? MR : s.rows, batch = LEAN ? 1 : s.batch;
    // PLAIN (with LEAN): no epilogue and no accumulation either -- the benchmark's product; carrying the two as
    // run-time values cost it 0.15 of its 12.4 us.
    static_assert(!PLAIN || LEAN, "PLAIN implies LEAN");
    const int epilogue = PLAIN ? (int)MNI_EPI_NONE : s.epilogue, accumulate = PLAIN ? 0 : s.accumulate;
    const int64_t o_cs = LEAN ? 1 : s.o_cs;
    const int x_bcount = LEAN ? 1 : s.x_bcount, w_bcount = LEAN ? 1 : s.w_bcount;
    __shared__ float4 red[SK_WAVES - 1][MR][64];
    const int ws_pitch = FUSED ? (s.cols + 31) & ~31 : s.cols;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    int group, slice, b, unit = 0;
    // A workgroup past the last unit is not turned away here but given an empty
    // K range and dismissed after the loop: an early return would make the
    // kernel wait for one kernel-argument fetch before it may start the next.
    bool alive = true;
    if (FUSED) {
        // grid = (units rounded up to a multiple of the XCD count, slices):
        // workgroups are dealt to XCDs by linear id, so unit u stays on XCD
        // u % xcds in every slice row of the grid.
        unit = blockIdx.x;
        slice = blockIdx.y;
        alive = unit < s.groups * batch;
        if (batch == 1) { b = 0; group = unit; }
        else { b = unit / s.groups; group = unit - b * s.groups; }
    } else {
        group = blockIdx.x; slice = blockIdx.y; b = blockIdx.z;
    }
    const int col0 = group * SK_COLS + 4 * lane;
    const int k_begin = slice * s.k_per_slice;
    const int k_end = alive ? min(s.K, k_begin + s.k_per_slice) : k_begin;
    const bool col_ok = LEAN || col0 < s.cols;  // cols % 4 == 0 is a launch precondition

    const int xb = x_bcount > 1 ? b % x_bcount : 0, wb = w_bcount > 1 ? b % w_bcount : 0;
    const float *__restrict__ X = s.X + (int64_t)xb * s.x_bs;
    const float *__restrict__ W = s.W + (int64_t)wb * s.w_bs + (col_ok ? col0 : 0);

    float4 acc[MR];
#pragma unroll
    for (int i = 0; i < MR; ++i) acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);

    // Decode shape: the bias (and, when nothing but a sum follows, the old output of an accumulating call) joins
    // the sum as part of the first K slice's partial.  That workgroup is dispatched first and is done long before
    // the reducers need its partial, so the loads cost nothing; asked for by the reducers -- whose own slices are
    // the last to finish -- they put a dependent round trip (0.85 us for one row) at the end of the kernel.
    const bool lean_activation = LEAN && epilogue >= MNI_EPI_BIAS_RELU;
    if (LEAN && slice == 0 && wave == 0 && alive) {
        if (epilogue != MNI_EPI_NONE) {
            float bv[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) bv[e] = s.bias[col0 + e];
#pragma unroll
            for (int i = 0; i < MR; ++i) acc[i] = make_float4(bv[0], bv[1], bv[2], bv[3]);
        }
        if (accumulate && !lean_activation) {
#pragma unroll
            for (int i = 0; i < MR; ++i) {
                const float4 old = *reinterpret_cast<const float4 *>(s.out + (int64_t)i * s.o_rs + col0);
                acc[i].x += old.x; acc[i].y += old.y; acc[i].z += old.z; acc[i].w += old.w;
            }
        }
    }

    for (int k0 = k_begin + wave * U; k0 < k_end; k0 += SK_WAVES * U) {
        f32x4 w[U];
        if (!TAIL || k0 + U <= k_end) {
            // whole group inside the slice: no clamps, no guards
            const float *__restrict__ wp = W + (int64_t)k0 * s.w_rs;
#pragma unroll
            for (int u = 0; u < U; ++u)
                w[u] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(wp + (int64_t)u * s.w_rs));
            // X is requested four rows at a time without looking at rows
            // (rows past it re-read the last row and are never stored):
            // guarding each row would put one scalar-load round trip after
            // the other.
#pragma unroll
            for (int i0 = 0; i0 < MR; i0 += 4) {
                float xv[4][U];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (i0 + i >= MR) continue;  // (MR need not be a multiple of 4)
                    const int ii = min(i0 + i, rows - 1);
                    if (XC) {  // X rows contiguous along k: one scalar load of U floats
                        const float *__restrict__ xr = X + (int64_t)ii * s.x_rs + k0;
#pragma unroll
                        for (int u = 0; u < U; ++u) xv[i][u] = xr[u];
                    } else {
                        const float *__restrict__ xr = X + (int64_t)ii * s.x_rs + (int64_t)k0 * s.x_cs;
#pragma unroll
                        for (int u = 0; u < U; ++u) xv[i][u] = xr[(int64_t)u * s.x_cs];
                    }
                }
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (i0 + i >= MR) continue;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        acc[i0 + i].x += xv[i][u] * w[u].x;
                        acc[i0 + i].y += xv[i][u] * w[u].y;
                        acc[i0 + i].z += xv[i][u] * w[u].z;
                        acc[i0 + i].w += xv[i][u] * w[u].w;
                    }
                }
            }
        } else if (TAIL) {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                // rows past the slice re-read its last row and meet x == 0
                const int krow = min(k0 + u, k_end - 1);
                w[u] = *reinterpret_cast<const f32x4 *>(W + (int64_t)krow * s.w_rs);
            }
#pragma unroll
            for (int i = 0; i < MR; ++i) {
                if (i < rows) {
                    const float *__restrict__ xr = X + (int64_t)i * s.x_rs + (int64_t)k0 * s.x_cs;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const float xv = (k0 + u < k_end) ? xr[(int64_t)u * s.x_cs] : 0.0f;
                        acc[i].x += xv * w[u].x;
                        acc[i].y += xv * w[u].y;
                        acc[i].z += xv * w[u].z;
                        acc[i].w += xv * w[u].w;
                    }
                }
            }
        }
    }

    if (FUSED && !alive) return;

    // ---- sum the wavefronts in wave order -------------------------------------
    if (wave > 0) {
#pragma unroll
        for (int i = 0; i < MR; ++i) red[wave - 1][i][lane] = acc[i];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int i = 0; i < MR; ++i) {
#pragma unroll
            for (int w = 0; w < SK_WAVES - 1; ++w) {
                const float4 p = red[w][i][lane];
                acc[i].x += p.x; acc[i].y += p.y; acc[i].z += p.z; acc[i].w += p.w;
            }
        }
        if (s.split_k > 1 && col_ok) {
            float *ws = s.ws + (((int64_t)slice * batch + b) * rows) * (int64_t)ws_pitch + col0;
#pragma unroll
            for (int i = 0; i < MR; ++i)
                if (i < rows) *reinterpret_cast<float4 *>(ws + (int64_t)i * ws_pitch) = acc[i];
        }
    }

    if (FUSED) {
        unsigned *flags = s.flags + (int64_t)unit * s.split_k;
        if (wave == 0) {
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the partial has reached L2
            if (lane == 0) flags[slice] = s.epoch;
        }
        const int reducers = min(min(rows, s.split_k), s.max_reducers);
        const int q = s.split_k - 1 - slice;
        if (q >= reducers) return;

        // Every wavefront of a reducer polls on its own (lane l watches slices l, l + 64, ...).
        bool arrived = false;
        for (int spin = 0; spin < SK_SPIN_LIMIT && !arrived; ++spin) {
            bool all = true;
            for (int s0 = 0; s0 < s.split_k; s0 += 64) {
                const int sl = s0 + lane;
                const unsigned v = sl < s.split_k ? sk_load_flag(flags + sl) : s.epoch;
                all = all && v == s.epoch;
            }
            arrived = __all(all);
            if (!arrived) __builtin_amdgcn_s_sleep(2);
        }
        // The partials are read with ordinary loads.  That is safe because no
        // 128-byte line of the workspace is shared by two units: its row pitch
        // is a whole number of lines (ws_pitch), so this CU's L1 cannot hold a
        // line of this unit from before its partials landed.

        constexpr int TB = 16;  // partials in flight per lane
        const int64_t slice_stride = (int64_t)batch * rows * ws_pitch;
        for (int row = q; row < rows; row += reducers) {
            f32x4 t = {0.f, 0.f, 0.f, 0.f};
            if (!arrived) {
                // NaN into the output and a code into the status word: the next call that
                // waits for the stream fails with it
                const float nan = __builtin_nanf("");
                t = f32x4{nan, nan, nan, nan};
                if (tid == 0) *s.status = DEVICE_STATUS_SKINNY_WAIT;
            } else if (col_ok) {
                const float *p = s.ws + ((int64_t)b * rows + row) * (int64_t)ws_pitch + col0;
                for (int s0 = wave; s0 < s.split_k; s0 += SK_WAVES * TB) {
                    f32x4 v[TB];
#pragma unroll
                    for (int j = 0; j < TB; ++j) {
                        const int sl = s0 + j * SK_WAVES;
                        v[j] = sl < s.split_k ? *reinterpret_cast<const f32x4 *>(p + (int64_t)sl * slice_stride)
                                              : f32x4{0.f, 0.f, 0.f, 0.f};
                    }
#pragma unroll
                    for (int j = 0; j < TB; ++j) t += v[j];
                }
            }
            __syncthreads();  // red is free again
            if (wave > 0) red[wave - 1][0][lane] = make_float4(t.x, t.y, t.z, t.w);
            __syncthreads();
            if (wave == 0 && col_ok) {
                float r[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
                for (int w = 0; w < SK_WAVES - 1; ++w) {
                    const float4 pw = red[w][0][lane];
                    r[0] += pw.x; r[1] += pw.y; r[2] += pw.z; r[3] += pw.w;
                }
                float *out = s.out + (int64_t)b * s.o_bs;
                if (LEAN) {
                    float4 *dst = reinterpret_cast<float4 *>(out + (int64_t)row * s.o_rs + col0);
                    if (lean_activation) {  // (the bias came in with the first slice's partial)
#pragma unroll
                        for (int e = 0; e < 4; ++e) r[e] = sk_epilogue(r[e], 0.0f, epilogue);
                        if (accumulate) {
                            const float4 old = *dst;
                            r[0] += old.x; r[1] += old.y; r[2] += old.z; r[3] += old.w;
                        }
                    }
                    *dst = make_float4(r[0], r[1], r[2], r[3]);
                    continue;
                }
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (epilogue != MNI_EPI_NONE)
                        r[e] = sk_epilogue(r[e], s.bias[s.bias_on_rows ? row : col0 + e], epilogue);
                    float *dst = out + (int64_t)row * s.o_rs + (int64_t)(col0 + e) * o_cs;
                    *dst = accumulate ? r[e] + *dst : r[e];
                }
            }
        }
        return;
    }

    if (wave != 0 || !col_ok || s.split_k > 1) return;
    float *out = s.out + (int64_t)b * s.o_bs;
#pragma unroll
    for (int i = 0; i < MR; ++i) {
        if (i < rows) {
            float r[4] = {acc[i].x, acc[i].y, acc[i].z, acc[i].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (epilogue != MNI_EPI_NONE) r[e] = sk_epilogue(r[e], s.bias[s.bias_on_rows ? i : col0 + e], epilogue);
                float *dst = out + (int64_t)i * s.o_rs + (int64_t)(col0 + e) * o_cs;
                *dst = accumulate ? r[e] + *dst : r[e];
            }
        }
    }
}

// Sums the K-slice partials ws[slice][batch][rows][cols] of a skinny product.
// The outputs are few and the slices many, so a workgroup of 16 wavefronts
// takes 64 outputs and spreads the slices over its wavefronts (wavefront g adds
// slices g, g + 16, ... in order, up to 4 loads in flight); the 16 sums are then
// combined in wavefront order.  The grouping depends only on the slice count,
// so the result is reproducible.
static constexpr int RED_GROUPS = 16;
__global__ __launch_bounds__(64 * RED_GROUPS) void skinny_reduce_kernel(const ReduceLaunch r) {
    __shared__ float sh[RED_GROUPS][64];
    const int lane = threadIdx.x & 63, g = threadIdx.x >> 6;
    const int64_t per_batch = (int64_t)r.rows * r.cols;
    const int64_t total = per_batch * r.batch;
    const int64_t idx = (int64_t)blockIdx.x * 64 + lane;
    float t = 0.0f;
    if (idx < total) {
        const float *p = r.ws + idx;
        int sl = g;
        for (; sl + 3 * RED_GROUPS < r.slices; sl += 4 * RED_GROUPS) {
            const float a = p[(int64_t)sl * total], b = p[(int64_t)(sl + RED_GROUPS) * total];
            const float c = p[(int64_t)(sl + 2 * RED_GROUPS) * total], d = p[(int64_t)(sl + 3 * RED_GROUPS) * total];
            t += a; t += b; t += c; t += d;
        }
        for (; sl < r.slices; sl += RED_GROUPS) t += p[(int64_t)sl * total];
    }
    sh[g][lane] = t;
    __syncthreads();
    if (g != 0 || idx >= total) return;
    float v = sh[0][lane];
#pragma unroll
    for (int k = 1; k < RED_GROUPS; ++k) v += sh[k][lane];
    const int b = (int)(idx / per_batch);
    const int64_t rem = idx - (int64_t)b * per_batch;
    const int i = (int)(rem / r.cols), j = (int)(rem - (int64_t)i * r.cols);
    if (r.epilogue != MNI_EPI_NONE) v = sk_epilogue(v, r.bias[r.bias_on_rows ? i : j], r.epilogue);
    float *dst = r.out + (int64_t)b * r.o_bs + (int64_t)i * r.o_rs + (int64_t)j * r.o_cs;
    if (r.accumulate) v += *dst;
    *dst = v;
}

// ---- W contiguous along K ------------------------------------------------------
// One wavefront per 4 output columns: lanes stride K with 16-byte loads of X
// and of the 4 W columns, then a butterfly reduction across the wavefront.
template <int MR>
__global__ __launch_bounds__(256) void skinny_dots_kernel(const SkinnyLaunch s) {
    constexpr int JW = 4;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int j0 = (blockIdx.x * 4 + wave) * JW;
    const int b = blockIdx.y;
    if (j0 >= s.cols) return;

    const float *__restrict__ X = s.X + (int64_t)(b % s.x_bcount) * s.x_bs;
    const float *__restrict__ W = s.W + (int64_t)(b % s.w_bcount) * s.w_bs;
    const float *wp[JW];
#pragma unroll
    for (int c = 0; c < JW; ++c) wp[c] = W + (int64_t)min(j0 + c, s.cols - 1) * s.w_cs;

    float acc[MR][JW];
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int c = 0; c < JW; ++c) acc[i][c] = 0.0f;

    for (int k = 4 * lane; k < s.K; k += 256) {  // K % 4 == 0 is a launch precondition
        float4 w[JW];
#pragma unroll
        for (int c = 0; c < JW; ++c) w[c] = *reinterpret_cast<const float4 *>(wp[c] + k);
#pragma unroll
        for (int i = 0; i < MR; ++i) {
            const int ii = i < s.rows ? i : 0;
            const float4 x = *reinterpret_cast<const float4 *>(X + (int64_t)ii * s.x_rs + k);
#pragma unroll
            for (int c = 0; c < JW; ++c)
                acc[i][c] += x.x * w[c].x + x.y * w[c].y + x.z * w[c].z + x.w * w[c].w;
        }
    }
#pragma unroll
    for (int i = 0; i < MR; ++i)
#pragma unroll
        for (int c = 0; c < JW; ++c) {
            float v = acc[i][c];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
            acc[i][c] = v;
        }
    if (lane != 0) return;
    float *out = s.out + (int64_t)b * s.o_bs;
#pragma unroll
    for (int i = 0; i < MR; ++i) {
        if (i >= s.rows) continue;
#pragma unroll
        for (int c = 0; c < JW; ++c) {
            const int j = j0 + c;
            if (j >= s.cols) continue;
            float *dst = out + (int64_t)i * s.o_rs + (int64_t)j * s.o_cs;
            float r = acc[i][c];
            if (s.epilogue != MNI_EPI_NONE) r = sk_epilogue(r, s.bias[s.bias_on_rows ? i : j], s.epilogue);
            if (s.accumulate) r += *dst;
            *dst = r;
        }
    }
}

// ---- split-K reduction ---------------------------------------------------------
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const ReduceLaunch r) {
    const int64_t per_batch = (int64_t)r.rows * r.cols;
    const int64_t total = per_batch * r.batch;
    const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    float v = 0.0f;
    for (int sl = 0; sl < r.slices; ++sl) v += r.ws[(int64_t)sl * total + idx];
    const int b = (int)(idx / per_batch);
    const int64_t rem = idx - (int64_t)b * per_batch;
    const int i = (int)(rem / r.cols), j = (int)(rem - (int64_t)i * r.cols);
    if (r.epilogue != MNI_EPI_NONE) v = sk_epilogue(v, r.bias[r.bias_on_rows ? i : j], r.epilogue);
    float *dst = r.out + (int64_t)b * r.o_bs + (int64_t)i * r.o_rs + (int64_t)j * r.o_cs;
    if (r.accumulate) v += *dst;
    *dst = v;
}

// The same, four adjacent columns per thread and four slices' loads in flight together (the sum of each element
// still runs in slice order: same value).  cols % 4 == 0, output rows contiguous and 16-byte aligned.
__global__ __launch_bounds__(256) void splitk_reduce4_kernel(const ReduceLaunch r) {
    const int64_t per_batch = (int64_t)r.rows * r.cols;
    const int64_t total4 = per_batch * r.batch / 4;
    const int64_t idx4 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx4 >= total4) return;
    const f32x4 *p = reinterpret_cast<const f32x4 *>(r.ws) + idx4;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    int sl = 0;
    for (; sl + 4 <= r.slices; sl += 4) {
        const f32x4 x0 = p[(int64_t)sl * total4], x1 = p[(int64_t)(sl + 1) * total4], x2 = p[(int64_t)(sl + 2) * total4],
                    x3 = p[(int64_t)(sl + 3) * total4];
        v += x0; v += x1; v += x2; v += x3;
    }
    for (; sl < r.slices; ++sl) v += p[(int64_t)sl * total4];
    const int64_t idx = 4 * idx4;
    const int b = (int)(idx / per_batch);
    const int64_t rem = idx - (int64_t)b * per_batch;
    const int i = (int)(rem / r.cols), j = (int)(rem - (int64_t)i * r.cols);
    float o[4] = {v.x, v.y, v.z, v.w};
    if (r.epilogue != MNI_EPI_NONE) {
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = sk_epilogue(o[e], r.bias[r.bias_on_rows ? i : j + e], r.epilogue);
    }
    f32x4 *dst = reinterpret_cast<f32x4 *>(r.out + (int64_t)b * r.o_bs + (int64_t)i * r.o_rs + j);
    if (r.accumulate) {
        const f32x4 old = *dst;
        o[0] += old.x; o[1] += old.y; o[2] += old.z; o[3] += old.w;
    }
    *dst = f32x4{o[0], o[1], o[2], o[3]};
}

int skinny_cols_block_cols() { return SK_COLS; }
int skinny_cols_rows_per_pass() { return SK_WAVES * SK_UNROLL; }

// The decode shape, for which the single-launch form has an instantiation per row count (1 to 8, and 16): X rows
// contiguous, K in whole groups of SK_UNROLL rows, one batch, whole 256-column groups, row-major 16-byte aligned
// output, the bias (if any) one value per column.
static bool skinny_decode_shape(const SkinnyLaunch &s) {
    return s.x_cs == 1 && s.K % SK_UNROLL == 0 && s.batch == 1 && (s.rows <= 8 || s.rows == 16) && s.cols % SK_COLS == 0 &&
           s.o_cs == 1 && s.o_rs % 4 == 0 && (reinterpret_cast<uintptr_t>(s.out) & 15) == 0 && !s.bias_on_rows &&
           s.epilogue <= MNI_EPI_BIAS_GELU;
}
#define MNI_SK_DECODE_ROWS(X) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(16)

template <int MR>
static void launch_skinny_cols_mr(const SkinnyLaunch &s, dim3 grid, bool fused) {
    const dim3 block(SK_THREADS);
    hipStream_t st = ctx().stream;
    const int variant = (s.x_cs == 1 ? 4 : 0) | (fused ? 2 : 0) | (s.K % SK_UNROLL != 0 ? 1 : 0);
    if (fused && skinny_decode_shape(s)) {
        const bool plain = s.epilogue == MNI_EPI_NONE && !s.accumulate;
        switch (s.rows) {
#define MNI_SK_LEAN(R) \
    case R: \
        if (plain) MNI_KERNEL_LAUNCH((skinny_cols_kernel<R, true, true, false, true, true>), grid, block, 0, st, s); \
        else MNI_KERNEL_LAUNCH((skinny_cols_kernel<R, true, true, false, true>), grid, block, 0, st, s); \
        return;
            MNI_SK_DECODE_ROWS(MNI_SK_LEAN)
#undef MNI_SK_LEAN
        }
    }
    switch (variant) {
#define MNI_SK(V, XC, FUSED, TAIL) \
    case V: MNI_KERNEL_LAUNCH((skinny_cols_kernel<MR, XC, FUSED, TAIL, false>), grid, block, 0, st, s); break;
        MNI_SK(0, false, false, false) MNI_SK(1, false, false, true)
        MNI_SK(2, false, true, false)  MNI_SK(3, false, true, true)
        MNI_SK(4, true, false, false)  MNI_SK(5, true, false, true)
        MNI_SK(6, true, true, false)   MNI_SK(7, true, true, true)
#undef MNI_SK
    }
}

int skinny_ws_pitch(int cols, bool single_launch) { return single_launch ? (cols + 31) & ~31 : cols; }

// How many workgroups of the single-launch form that `s` would run as fit one CU together (what the runtime's
// occupancy calculation says for that instantiation: between 1 for the 16-row general form, whose 253 VGPRs
// leave room for one wavefront per SIMD, and 6).  0 if the query fails.
template <int MR>
static int skinny_cols_fused_occupancy_mr(const SkinnyLaunch &s) {
    const int variant = (s.x_cs == 1 ? 4 : 0) | 2 | (s.K % SK_UNROLL != 0 ? 1 : 0);
    if (skinny_decode_shape(s)) {  // (the rule of launch_skinny_cols_mr)
        static int by_rows[17] = {-1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1, -1};
        if (by_rows[s.rows] < 0) {
            int n = 0;
            hipError_t e = hipErrorInvalidValue;
            switch (s.rows) {
#define MNI_SK_LEAN(R) \
    case R: e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, skinny_cols_kernel<R, true, true, false, true>, SK_THREADS, 0); break;  /* (the plain form needs no more) */
                MNI_SK_DECODE_ROWS(MNI_SK_LEAN)
#undef MNI_SK_LEAN
            }
            if (e != hipSuccess) { (void)hipGetLastError(); n = 0; }
            by_rows[s.rows] = n;
        }
        return by_rows[s.rows];
    }
    static int cache[4] = {-1, -1, -1, -1};  // per (x contiguous, tail)
    const int slot = (variant & 4 ? 2 : 0) | (variant & 1);
    if (cache[slot] < 0) {
        int n = 0;
        hipError_t e;
        if (slot == 0) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, skinny_cols_kernel<MR, false, true, false, false>, SK_THREADS, 0);
        else if (slot == 1) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, skinny_cols_kernel<MR, false, true, true, false>, SK_THREADS, 0);
        else if (slot == 2) e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, skinny_cols_kernel<MR, true, true, false, false>, SK_THREADS, 0);
        else e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, skinny_cols_kernel<MR, true, true, true, false>, SK_THREADS, 0);
        if (e != hipSuccess) { (void)hipGetLastError(); n = 0; }
        cache[slot] = n;
    }
    return cache[slot];
}
int skinny_cols_fused_occupancy(const SkinnyLaunch &s) {
    if (s.rows <= 4) return skinny_cols_fused_occupancy_mr<4>(s);
    if (s.rows <= 8) return skinny_cols_fused_occupancy_mr<8>(s);
    if (s.rows <= 16) return skinny_cols_fused_occupancy_mr<16>(s);
    return 0;
}

int launch_skinny_cols(const SkinnyLaunch &s, int xcds) {
    if (s.rows <= 0 || s.cols <= 0 || s.batch <= 0) return MNI_OK;
    const int groups = (s.cols + SK_COLS - 1) / SK_COLS;
    if (s.groups != groups) return set_error(MNI_ERR_INVALID, "skinny launch: column group count not set");
    if (s.k_per_slice % SK_UNROLL != 0 && s.split_k > 1)
        return set_error(MNI_ERR_INVALID, "skinny launch: a K slice must be whole groups of %d rows", SK_UNROLL);
    const bool fused = xcds > 0 && s.split_k > 1;
    dim3 grid(groups, s.split_k, s.batch);
    if (fused) {
        if (!s.flags || !s.ws || !s.status) return set_error(MNI_ERR_INVALID, "single-launch skinny product without flags/partials");
        const int64_t units = (int64_t)groups * s.batch;
        grid = dim3((unsigned)((units + xcds - 1) / xcds * xcds), s.split_k);
    }
    if (s.rows <= 4) launch_skinny_cols_mr<4>(s, grid, fused);
    else if (s.rows <= 8) launch_skinny_cols_mr<8>(s, grid, fused);
    else if (s.rows <= 16) launch_skinny_cols_mr<16>(s, grid, fused);
    else return set_error(MNI_ERR_INVALID, "skinny kernel takes at most 16 rows, got %d", s.rows);
    return check_launch("skinny_cols_kernel");
}

int launch_skinny_reduce(const ReduceLaunch &r) {
    const int64_t total = (int64_t)r.rows * r.cols * r.batch;
    if (total <= 0) return MNI_OK;
    MNI_KERNEL_LAUNCH(skinny_reduce_kernel, dim3((unsigned)((total + 63) / 64)), dim3(64 * RED_GROUPS), 0, ctx().stream, r);
    return check_launch("skinny_reduce_kernel");
}

int launch_skinny_dots(const SkinnyLaunch &s) {
    if (s.rows <= 0 || s.cols <= 0 || s.batch <= 0) return MNI_OK;
    dim3 grid((s.cols + 15) / 16, s.batch), block(256);
    hipStream_t st = ctx().stream;
    if (s.rows <= 4) MNI_KERNEL_LAUNCH((skinny_dots_kernel<4>), grid, block, 0, st, s);
    else if (s.rows <= 8) MNI_KERNEL_LAUNCH((skinny_dots_kernel<8>), grid, block, 0, st, s);
    else if (s.rows <= 16) MNI_KERNEL_LAUNCH((skinny_dots_kernel<16>), grid, block, 0, st, s);
    else return set_error(MNI_ERR_INVALID, "skinny kernel takes at most 16 rows, got %d", s.rows);
    return check_launch("skinny_dots_kernel");
}

int launch_splitk_reduce(const ReduceLaunch &r) {
    const int64_t total = (int64_t)r.rows * r.cols * r.batch;
    if (total <= 0) return MNI_OK;
    const bool by4 = r.cols % 4 == 0 && r.o_cs == 1 && r.o_rs % 4 == 0 && r.o_bs % 4 == 0 && (reinterpret_cast<uintptr_t>(r.out) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(r.ws) & 15) == 0;
    dim3 block(256);
    if (by4) {
        MNI_KERNEL_LAUNCH(splitk_reduce4_kernel, dim3((unsigned)((total / 4 + 255) / 256)), block, 0, ctx().stream, r);
        return check_launch("splitk_reduce4_kernel");
    }
    dim3 grid((unsigned)((total + 255) / 256));
    MNI_KERNEL_LAUNCH(splitk_reduce_kernel, grid, block, 0, ctx().stream, r);
    return check_launch("splitk_reduce_kernel");
}

}  // namespace mni
