// Yardsticks, timed the way mni_rocm_sgemm_timed times products: an empty
// launch, a pure read, a pure write and a copy of a caller-supplied buffer, and
// a loop of nothing but MFMAs.  They say what this device gives a kernel that does nothing but
// stream -- the figure a bandwidth-bound product (the skinny kernels, the
// batched attention-shaped products) is to be held against, next to the
// datasheet's.  No counterpart in the reference.
#include "common.h"

namespace mni {

typedef float f32x4 __attribute__((ext_vector_type(4)));
static constexpr int YS_THREADS = 256;
static constexpr int YS_UNROLL = 8;  // 16-byte pieces in flight per lane

__global__ void ys_empty_kernel() {}

// Every workgroup streams a contiguous run of 16-byte pieces; a lane keeps
// YS_UNROLL requests in flight.  The values are folded into one float that is
// stored only if it equals a value no finite input produces, so the loads
// cannot be dropped and nothing is written.
template <bool NT>
__global__ __launch_bounds__(YS_THREADS) void ys_read_kernel(const f32x4 *__restrict__ src, int64_t n4, float *sink) {
    const int64_t per_block = (n4 + gridDim.x - 1) / gridDim.x;
    const int64_t lo = (int64_t)blockIdx.x * per_block, hi = min(n4, lo + per_block);
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
    int64_t p = lo + threadIdx.x;
    for (; p + (YS_UNROLL - 1) * YS_THREADS < hi; p += YS_UNROLL * YS_THREADS) {
        f32x4 v[YS_UNROLL];
#pragma unroll
        for (int u = 0; u < YS_UNROLL; ++u)
            v[u] = NT ? __builtin_nontemporal_load(src + p + u * YS_THREADS) : src[p + u * YS_THREADS];
#pragma unroll
        for (int u = 0; u < YS_UNROLL; ++u) s += v[u];
    }
    for (; p < hi; p += YS_THREADS) s += src[p];
    const float t = (s.x + s.y) + (s.z + s.w);
    if (t == -1.2345678e38f) *sink = t;
}

template <bool NT>
__global__ __launch_bounds__(YS_THREADS) void ys_write_kernel(f32x4 *__restrict__ dst, int64_t n4, float value) {
    const int64_t per_block = (n4 + gridDim.x - 1) / gridDim.x;
    const int64_t lo = (int64_t)blockIdx.x * per_block, hi = min(n4, lo + per_block);
    const f32x4 v = {value, value, value, value};
    for (int64_t p = lo + threadIdx.x; p < hi; p += YS_THREADS) {
        if (NT) __builtin_nontemporal_store(v, dst + p);
        else dst[p] = v;
    }
}

template <bool NT>
__global__ __launch_bounds__(YS_THREADS) void ys_copy_kernel(f32x4 *__restrict__ dst, const f32x4 *__restrict__ src, int64_t n4) {
    const int64_t per_block = (n4 + gridDim.x - 1) / gridDim.x;
    const int64_t lo = (int64_t)blockIdx.x * per_block, hi = min(n4, lo + per_block);
    int64_t p = lo + threadIdx.x;
    for (; p + (YS_UNROLL - 1) * YS_THREADS < hi; p += YS_UNROLL * YS_THREADS) {
        f32x4 v[YS_UNROLL];
#pragma unroll
        for (int u = 0; u < YS_UNROLL; ++u)
            v[u] = NT ? __builtin_nontemporal_load(src + p + u * YS_THREADS) : src[p + u * YS_THREADS];
#pragma unroll
        for (int u = 0; u < YS_UNROLL; ++u) {
            if (NT) __builtin_nontemporal_store(v[u], dst + p + u * YS_THREADS);
            else dst[p + u * YS_THREADS] = v[u];
        }
    }
    for (; p < hi; p += YS_THREADS) dst[p] = src[p];
}

// What the matrix pipe gives a loop of nothing but fp32 MFMAs, and what it
// still gives when every MFMA is followed by VALU vector-ALU instructions that
// depend on nothing: on this chip the fp32 MFMA and the vector ALU share issue
// time, so the second figure is what any kernel pays per address computation or
// register move inside its MFMA loop.  Four independent accumulators per
// wavefront (an MFMA never waits for the one before it).
typedef float floatx16 __attribute__((ext_vector_type(16)));

template <int VALU>
__global__ __launch_bounds__(YS_THREADS) void ys_mfma_kernel(float *sink, int rounds) {
    floatx16 acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][e] = 0.f;
    const float a = threadIdx.x * 1e-6f, b = blockIdx.x * 1e-6f;
    float x = a, y = b;
    for (int it = 0; it < rounds; ++it) {
#pragma unroll
        for (int rep = 0; rep < 4; ++rep)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[i], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int v = 0; v < VALU; ++v) asm volatile("v_mov_b32 %0, %1" : "=v"(x) : "v"(y));
                __builtin_amdgcn_sched_barrier(0);
            }
    }
    float s = x;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) s += acc[i][e];
    if (s == -1.2345678e38f) *sink = s;
}

}  // namespace mni

using namespace mni;

extern "C" int mni_rocm_mfma_yardstick_timed(int valu_per_mfma, int waves_per_simd, int mfmas_per_wave, int warmup, int iters, float *avg_ms) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    if (valu_per_mfma < 0 || valu_per_mfma > 2 || waves_per_simd < 1 || waves_per_simd > 2 || mfmas_per_wave < 16 || mfmas_per_wave % 16 != 0 ||
        iters <= 0 || warmup < 0 || !avg_ms)
        return set_error(MNI_ERR_INVALID, "mfma yardstick: bad arguments");
    DeviceCtx &c = ctx();
    const dim3 grid((unsigned)((c.compute_units > 0 ? c.compute_units : 256) * waves_per_simd)), block(YS_THREADS);
    float *sink = (float *)c.skinny_flags;  // never written
    const int rounds = mfmas_per_wave / 16;
    auto launch = [&]() {
        if (valu_per_mfma == 0) MNI_KERNEL_LAUNCH((ys_mfma_kernel<0>), grid, block, 0, c.stream, sink, rounds);
        else if (valu_per_mfma == 1) MNI_KERNEL_LAUNCH((ys_mfma_kernel<1>), grid, block, 0, c.stream, sink, rounds);
        else MNI_KERNEL_LAUNCH((ys_mfma_kernel<2>), grid, block, 0, c.stream, sink, rounds);
    };
    for (int i = 0; i < warmup; ++i) launch();
    MNI_TRY(check_launch("mfma yardstick"));
    hipEvent_t e0, e1;
    MNI_HIP_CHECK(hipEventCreate(&e0));
    MNI_HIP_CHECK(hipEventCreate(&e1));
    hipError_t he = hipEventRecord(e0, c.stream);
    for (int i = 0; i < iters; ++i) launch();
    if (he == hipSuccess) he = hipEventRecord(e1, c.stream);
    if (he == hipSuccess) he = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (he != hipSuccess) return set_error(MNI_ERR_HIP, "mfma yardstick: %s", hipGetErrorString(he));
    MNI_TRY(check_launch("mfma yardstick"));
    *avg_ms = ms / (float)iters;
    return MNI_OK;
}

extern "C" int mni_rocm_yardstick_timed(int kind, int nontemporal, void *dst, const void *const *srcs, int nsrc, size_t bytes,
                                        int blocks_per_cu, int warmup, int iters, float *avg_ms) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    if (kind < MNI_YARDSTICK_EMPTY || kind > MNI_YARDSTICK_COPY || iters <= 0 || warmup < 0 || !avg_ms || blocks_per_cu <= 0)
        return set_error(MNI_ERR_INVALID, "yardstick: bad arguments");
    const bool reads = kind == MNI_YARDSTICK_READ || kind == MNI_YARDSTICK_COPY;
    const bool writes = kind == MNI_YARDSTICK_WRITE || kind == MNI_YARDSTICK_COPY;
    if (kind != MNI_YARDSTICK_EMPTY) {
        if (bytes == 0 || bytes % 16 != 0) return set_error(MNI_ERR_INVALID, "yardstick: size must be a positive multiple of 16 bytes");
        if (reads && (!srcs || nsrc <= 0)) return set_error(MNI_ERR_INVALID, "yardstick: no source buffers");
        if (writes && !dst) return set_error(MNI_ERR_INVALID, "yardstick: no destination buffer");
        for (int i = 0; reads && i < nsrc; ++i)
            if (!srcs[i] || ((uintptr_t)srcs[i] & 15)) return set_error(MNI_ERR_INVALID, "yardstick: source %d is null or not 16-byte aligned", i);
        if (writes && ((uintptr_t)dst & 15)) return set_error(MNI_ERR_INVALID, "yardstick: destination is not 16-byte aligned");
    }
    DeviceCtx &c = ctx();
    const int64_t n4 = (int64_t)(bytes / 16);
    const dim3 grid((unsigned)((c.compute_units > 0 ? c.compute_units : 256) * blocks_per_cu)), block(YS_THREADS);
    float *sink = (float *)c.skinny_flags;  // never written: see ys_read_kernel
    auto launch = [&](int it) {
        const f32x4 *src = reads ? (const f32x4 *)srcs[it % nsrc] : nullptr;
        switch (kind) {
        case MNI_YARDSTICK_EMPTY: MNI_KERNEL_LAUNCH(ys_empty_kernel, dim3(1), dim3(64), 0, c.stream); break;
        case MNI_YARDSTICK_READ:
            if (nontemporal) MNI_KERNEL_LAUNCH((ys_read_kernel<true>), grid, block, 0, c.stream, src, n4, sink);
            else MNI_KERNEL_LAUNCH((ys_read_kernel<false>), grid, block, 0, c.stream, src, n4, sink);
            break;
        case MNI_YARDSTICK_WRITE:
            if (nontemporal) MNI_KERNEL_LAUNCH((ys_write_kernel<true>), grid, block, 0, c.stream, (f32x4 *)dst, n4, 1.0f);
            else MNI_KERNEL_LAUNCH((ys_write_kernel<false>), grid, block, 0, c.stream, (f32x4 *)dst, n4, 1.0f);
            break;
        default:
            if (nontemporal) MNI_KERNEL_LAUNCH((ys_copy_kernel<true>), grid, block, 0, c.stream, (f32x4 *)dst, src, n4);
            else MNI_KERNEL_LAUNCH((ys_copy_kernel<false>), grid, block, 0, c.stream, (f32x4 *)dst, src, n4);
        }
    };
    int it = 0;
    for (int i = 0; i < warmup; ++i) launch(it++);
    MNI_TRY(check_launch("yardstick"));
    hipEvent_t e0, e1;
    MNI_HIP_CHECK(hipEventCreate(&e0));
    MNI_HIP_CHECK(hipEventCreate(&e1));
    hipError_t he = hipEventRecord(e0, c.stream);
    for (int i = 0; i < iters; ++i) launch(it++);
    if (he == hipSuccess) he = hipEventRecord(e1, c.stream);
    if (he == hipSuccess) he = hipEventSynchronize(e1);
    float ms = 0.0f;
    if (he == hipSuccess) he = hipEventElapsedTime(&ms, e0, e1);
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (he != hipSuccess) return set_error(MNI_ERR_HIP, "yardstick: %s", hipGetErrorString(he));
    MNI_TRY(check_launch("yardstick"));
    *avg_ms = ms / (float)iters;
    return MNI_OK;
}
