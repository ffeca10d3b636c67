// Device singleton, caching allocator, copies and timing marks.
// Counterpart of the cuda arm's GpuDevice (src/native/src/device.rs:29-48) and
// CachingAllocator (src/native/src/allocator.rs:46-84) in the reference: one
// device, one stream, kernels prebuilt into this library.
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <atomic>
#include <chrono>

#include <unordered_map>
#include <vector>

#include "common.h"

namespace mni {

// Per thread, so that a message read after a failed call is that call's own.
static thread_local char g_err_shared[1024];

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err_shared, sizeof g_err_shared, fmt, ap);
    va_end(ap);
    return code;
}

std::recursive_mutex &api_mutex() {
    static std::recursive_mutex m;
    return m;
}

DeviceCtx &ctx() {
    static DeviceCtx c;
    return c;
}

// Workspace of mni_rocm_sgemm_noalloc, the entry point for callers that cannot
// allocate: the K-slice / stream-K partial sums of one product.  Part of the
// code object, so the device holds it from the moment the library is loaded
// until the process ends.  On the host this name is only a handle for
// hipGetSymbolAddress; the device address is looked up once in init_device and
// kept in the device context, and that address is what kernels are given.
static constexpr size_t NOALLOC_SCRATCH_BYTES = (size_t)32 << 20;
static __device__ __align__(256) float scratch[NOALLOC_SCRATCH_BYTES / sizeof(float)];

// Which XCD a workgroup runs on: the hardware id, read by one lane.
__global__ void xcc_probe_kernel(unsigned *out) {
    if (threadIdx.x == 0) {
        unsigned v;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(v));
        out[blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)] = v & 0xf;
    }
}

// Confirms that workgroups are dealt to the XCDs round-robin by linear id
// (x fastest; workgroup b on XCD b % count), also in a 2-D/3-D grid, which the
// single-launch skinny kernel relies on to keep a column group's partial sums
// inside one XCD's L2.
static int probe_xcd_mapping(DeviceCtx &c) {
    const dim3 grid(24, 29, 3);  // 24 = a multiple of 8 XCDs, as the skinny kernel's grids are
    constexpr int BLOCKS = 24 * 29 * 3;
    unsigned *dev = nullptr;
    MNI_HIP_CHECK(hipMalloc((void **)&dev, BLOCKS * sizeof(unsigned)));
    MNI_KERNEL_LAUNCH(xcc_probe_kernel, grid, dim3(64), 0, c.stream, dev);
    std::vector<unsigned> host(BLOCKS);
    hipError_t e = hipMemcpyAsync(host.data(), dev, BLOCKS * sizeof(unsigned), hipMemcpyDeviceToHost, c.stream);
    if (e == hipSuccess) e = hipStreamSynchronize(c.stream);
    (void)hipFree(dev);
    if (e != hipSuccess) return set_error(MNI_ERR_HIP, "XCD probe failed: %s", hipGetErrorString(e));
    unsigned count = 0;
    for (unsigned v : host) count = v + 1 > count ? v + 1 : count;
    bool round_robin = count > 0;
    for (int b = 0; b < BLOCKS && round_robin; ++b) round_robin = host[b] == (unsigned)b % count;
    c.xcd_count = round_robin ? (int)count : 0;
    return MNI_OK;
}

static int init_device(int device) {
    DeviceCtx &c = ctx();
    if (c.ready) {
        if (device != c.device)
            return set_error(MNI_ERR_INVALID, "library already initialised on device %d", c.device);
        return MNI_OK;
    }
    int count = 0;
    MNI_HIP_CHECK(hipGetDeviceCount(&count));
    if (device < 0 || device >= count)
        return set_error(MNI_ERR_INVALID, "device %d out of range (%d visible)", device, count);
    MNI_HIP_CHECK(hipSetDevice(device));
    hipDeviceProp_t prop;
    MNI_HIP_CHECK(hipGetDeviceProperties(&prop, device));
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return set_error(MNI_ERR_INVALID, "libmni_rocm is built for gfx950 only, found %s", prop.gcnArchName);
    c.device = device;
    c.compute_units = prop.multiProcessorCount;
    c.clock_khz = prop.clockRate;
    snprintf(c.name, sizeof c.name, "%s (%s)", prop.name, prop.gcnArchName);
    // Default priority on purpose: streams of mixed priority are avoided.
    MNI_HIP_CHECK(hipStreamCreateWithFlags(&c.stream, hipStreamNonBlocking));
    MNI_TRY(probe_xcd_mapping(c));
    c.skinny_flag_cap = 1 << 16;
    MNI_HIP_CHECK(hipMalloc((void **)&c.skinny_flags, c.skinny_flag_cap * sizeof(unsigned)));
    MNI_HIP_CHECK(hipMemset(c.skinny_flags, 0, c.skinny_flag_cap * sizeof(unsigned)));
    c.skinny_epoch = 0;
    c.fewrows_counter_cap = 4096;
    MNI_HIP_CHECK(hipMalloc((void **)&c.fewrows_counters, c.fewrows_counter_cap * sizeof(unsigned)));
    MNI_HIP_CHECK(hipMemset(c.fewrows_counters, 0, c.fewrows_counter_cap * sizeof(unsigned)));
    c.gemv_slot_cap = 256 * 512;  // one workgroup per CU, a tile of up to 32 rows x 64 columns (or 8 x 128) in 16-byte pieces
    MNI_HIP_CHECK(hipMalloc(&c.gemv_pa, c.gemv_slot_cap * 16));
    MNI_HIP_CHECK(hipMalloc(&c.gemv_pb, c.gemv_slot_cap * 8));
    MNI_HIP_CHECK(hipMemset(c.gemv_pa, 0, c.gemv_slot_cap * 16));
    MNI_HIP_CHECK(hipMemset(c.gemv_pb, 0, c.gemv_slot_cap * 8));
    c.gemv_counter_cap = 256 * 8;
    MNI_HIP_CHECK(hipMalloc((void **)&c.gemv_counters, c.gemv_counter_cap * sizeof(unsigned)));
    MNI_HIP_CHECK(hipMemset(c.gemv_counters, 0, c.gemv_counter_cap * sizeof(unsigned)));
    // Pinned staging slots of upload_small, and one event per slot that says when its transfer has left it.
    MNI_HIP_CHECK(hipHostMalloc((void **)&c.stage_host, DeviceCtx::STAGE_SLOTS * DeviceCtx::STAGE_BYTES, hipHostMallocDefault));
    for (int i = 0; i < DeviceCtx::STAGE_SLOTS; ++i) MNI_HIP_CHECK(hipEventCreateWithFlags(&c.stage_done[i], hipEventDisableTiming));
    // Pinned, device-visible host memory: a kernel writes the word over the
    // bus in the rare case it has something to report, the host reads it for
    // free after every wait.
    MNI_HIP_CHECK(hipHostMalloc((void **)&c.status_host, 64, hipHostMallocMapped));
    memset(c.status_host, 0, 64);
    MNI_HIP_CHECK(hipHostGetDevicePointer((void **)&c.status_dev, c.status_host, 0));
    MNI_HIP_CHECK(hipHostMalloc((void **)&c.fetch_host, DeviceCtx::STAGE_BYTES, hipHostMallocMapped));
    MNI_HIP_CHECK(hipHostGetDevicePointer((void **)&c.fetch_dev, c.fetch_host, 0));
    c.result_host = (unsigned long long *)(c.status_host + 2);  // bytes 8..15 of the block
    c.result_dev = (unsigned long long *)(c.status_dev + 2);
    // Device address of the static workspace on this device (the library drives one device).
    float *scratch_ptr = nullptr;
    MNI_HIP_CHECK(hipGetSymbolAddress((void **)&scratch_ptr, HIP_SYMBOL(scratch)));
    c.noalloc_scratch = scratch_ptr;
    c.noalloc_scratch_bytes = NOALLOC_SCRATCH_BYTES;
    c.ready = true;
    return MNI_OK;
}

int ensure_init() {
    if (ctx().ready) return MNI_OK;
    return init_device(0);
}

// Watches the result word for `tag` for at most `micros` microseconds.
static bool poll_result_word(unsigned tag, unsigned *value, int micros) {
    volatile unsigned long long *w = ctx().result_host;
    const auto t0 = std::chrono::steady_clock::now();
    for (;;) {
        for (int i = 0; i < 64; ++i) {
            const unsigned long long v = *w;
            if ((unsigned)(v >> 32) == tag) {
                if (value) *value = (unsigned)v;
                // what the kernel wrote to pinned memory before the tag is read by the caller after this
                std::atomic_thread_fence(std::memory_order_acquire);
                return true;
            }
            __builtin_ia32_pause();
        }
        if (std::chrono::steady_clock::now() - t0 > std::chrono::microseconds(micros)) return false;
    }
}
static int blocking_sync(const char *what) {
    MNI_HIP_CHECK(hipStreamSynchronize(ctx().stream));
    return check_device_status(what);
}
unsigned next_result_tag() {
    DeviceCtx &c = ctx();
    if (++c.result_seq == 0) ++c.result_seq;
    *(volatile unsigned long long *)c.result_host = 0;  // (every earlier result has been waited for)
    return c.result_seq;
}
int wait_result_word(unsigned tag, unsigned *value, bool *delivered) {
    *delivered = true;
    if (poll_result_word(tag, value, 200)) return MNI_OK;
    MNI_TRY(blocking_sync("waiting for a kernel's result"));
    *delivered = poll_result_word(tag, value, 0);
    return MNI_OK;
}

__global__ void marker_kernel(unsigned long long *word, unsigned tag) { post_result_word(word, tag, 0u); }
// Up to DeviceCtx::STAGE_BYTES of device memory into pinned host memory, then the tag.
__global__ __launch_bounds__(256) void fetch_small_kernel(unsigned *__restrict__ host, const unsigned *__restrict__ src, int words,
                                                          unsigned long long *word, unsigned tag) {
    for (int i = threadIdx.x; i < words; i += 256) host[i] = src[i];
    __threadfence_system();
    __syncthreads();
    if (threadIdx.x == 0) post_result_word(word, tag, 0u);
}

// The stream runs in order, so a one-thread kernel queued now runs when everything before it is done; it
// writes a tag to pinned host memory and the host watches for it.  That takes a few microseconds after the
// last kernel ends; the runtime's own wait queues a barrier and sleeps on an interrupt, some twenty more.  Work
// that lasts longer than the watch falls back on the runtime's wait.
int sync_stream_checked(const char *what) {
    DeviceCtx &c = ctx();
    const unsigned tag = next_result_tag();
    hipLaunchKernelGGL(marker_kernel, dim3(1), dim3(1), 0, c.stream, c.result_dev, tag);  // (not counted as a launch of the caller's work)
    if (hipGetLastError() == hipSuccess && poll_result_word(tag, nullptr, 150)) return check_device_status(what);
    return blocking_sync(what);
}

int check_device_status(const char *what) {
    DeviceCtx &c = ctx();
    if (!c.status_host) return MNI_OK;
    const unsigned st = *(volatile unsigned *)c.status_host;
    if (st == DEVICE_STATUS_OK) return MNI_OK;
    *(volatile unsigned *)c.status_host = DEVICE_STATUS_OK;
    const char *who = st == DEVICE_STATUS_STREAMK_WAIT  ? "gemm_mfma_kernel (stream-K): a finishing workgroup gave up waiting for a partial tile"
                      : st == DEVICE_STATUS_SKINNY_WAIT ? "skinny_cols_kernel: a reducing workgroup gave up waiting for a K-slice partial"
                      : st == DEVICE_STATUS_GEMV_WAIT   ? "gemv_units_kernel: the adding wavefront gave up waiting for a K-slice partial"
                                                        : "a kernel reported an unknown status";
    return set_error(MNI_ERR_HIP, "%s: device status %u -- %s; results written since the last synchronisation hold NaN where "
                                  "the wait expired", what, st, who);
}

int gemm_ws_alloc(void **p, size_t bytes) {
    DeviceCtx &c = ctx();
    if (!c.scratch) return dev_alloc(p, bytes);
    if (bytes > c.scratch_bytes)
        return set_error(MNI_ERR_INVALID, "sgemm_noalloc: this product needs %zu bytes of workspace, the fixed scratch holds %zu",
                         bytes, c.scratch_bytes);
    *p = c.scratch;
    return MNI_OK;
}
void gemm_ws_free(void *p) {
    if (p && p != (void *)ctx().scratch) dev_free(p);
}

int check_launch(const char *what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return set_error(MNI_ERR_HIP, "launch of %s failed: %s", what, hipGetErrorString(e));
    return MNI_OK;
}

// ---- allocator --------------------------------------------------------------
// Exact-size free lists keyed by the rounded request, like the reference's
// allocator; sizes are rounded up to 256 B so that every buffer is aligned for
// 16-byte vector access and small tensors share lists.
struct Allocator {
    std::unordered_map<size_t, std::vector<void *>> free_lists;
    std::unordered_map<void *, size_t> live;  // ptr -> rounded size
    size_t total = 0;
    size_t cached = 0;
    uint64_t requests = 0, driver_allocations = 0, releases = 0;  // dev_alloc calls, hipMalloc calls, dev_free calls
};
static Allocator &allocator() {
    // Never destroyed: tensors of the engine (another translation unit's
    // static) return their buffers here while the process exits, in an order
    // the language does not fix; the driver reclaims device memory itself.
    static Allocator *a = new Allocator;
    return *a;
}
static size_t round_size(size_t bytes) {
    if (bytes == 0) bytes = 4;
    return (bytes + 255) & ~(size_t)255;
}

int dev_alloc(void **p, size_t bytes) {
    MNI_TRY(ensure_init());
    Allocator &a = allocator();
    ++a.requests;
    size_t sz = round_size(bytes);
    auto it = a.free_lists.find(sz);
    if (it != a.free_lists.end() && !it->second.empty()) {
        *p = it->second.back();
        it->second.pop_back();
        a.cached -= sz;
        a.live[*p] = sz;
        return MNI_OK;
    }
    hipError_t e = hipMalloc(p, sz);
    if (e != hipSuccess) {
        // Give cached blocks back to the driver and retry once.
        (void)hipGetLastError();
        dev_clear_cache();
        e = hipMalloc(p, sz);
        if (e != hipSuccess) {
            (void)hipGetLastError();
            return set_error(MNI_ERR_NOMEM, "hipMalloc(%zu) failed: %s", sz, hipGetErrorString(e));
        }
    }
    ++a.driver_allocations;
    a.total += sz;
    a.live[*p] = sz;
    return MNI_OK;
}

int dev_free(void *p) {
    if (!p) return MNI_OK;
    Allocator &a = allocator();
    auto it = a.live.find(p);
    if (it == a.live.end()) return set_error(MNI_ERR_INVALID, "free of a pointer this library did not allocate");
    ++a.releases;
    a.free_lists[it->second].push_back(p);
    a.cached += it->second;
    a.live.erase(it);
    return MNI_OK;
}

int dev_clear_cache() {
    Allocator &a = allocator();
    bool any = false;
    for (auto &kv : a.free_lists) any = any || !kv.second.empty();
    if (!any) return MNI_OK;
    // Cached blocks may still be read by queued kernels.
    if (ctx().ready) MNI_HIP_CHECK(hipStreamSynchronize(ctx().stream));
    for (auto &kv : a.free_lists) {
        for (void *p : kv.second) {
            (void)hipFree(p);
            a.total -= kv.first;
        }
        kv.second.clear();
    }
    a.free_lists.clear();
    a.cached = 0;
    return MNI_OK;
}

size_t dev_cached_bytes() { return allocator().cached; }
void dev_alloc_stats(uint64_t *requests, uint64_t *driver_allocations, uint64_t *releases, uint64_t *cached_bytes) {
    const Allocator &a = allocator();
    *requests = a.requests; *driver_allocations = a.driver_allocations; *releases = a.releases; *cached_bytes = a.cached;
}

}  // namespace mni

using namespace mni;

namespace mni {
int upload_small(void *dst, const void *src, size_t bytes) {
    MNI_TRY(ensure_init());
    if (bytes == 0) return MNI_OK;
    DeviceCtx &c = ctx();
    if (bytes > DeviceCtx::STAGE_BYTES || !c.stage_host) return mni_rocm_h2d(dst, src, bytes);
    const unsigned slot = c.stage_next++ % DeviceCtx::STAGE_SLOTS;
    if (c.stage_used[slot]) MNI_HIP_CHECK(hipEventSynchronize(c.stage_done[slot]));  // sixteen uploads ago: long done
    char *host = c.stage_host + (size_t)slot * DeviceCtx::STAGE_BYTES;
    memcpy(host, src, bytes);
    MNI_HIP_CHECK(hipMemcpyAsync(dst, host, bytes, hipMemcpyHostToDevice, c.stream));
    MNI_HIP_CHECK(hipEventRecord(c.stage_done[slot], c.stream));
    c.stage_used[slot] = true;
    return MNI_OK;
}
}  // namespace mni

extern "C" {

int mni_rocm_init(int device) { MNI_API_GUARD; return init_device(device); }

int mni_rocm_device_info(char *name, size_t name_cap, int *compute_units, int *clock_khz) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    if (name && name_cap) snprintf(name, name_cap, "%s", ctx().name);
    if (compute_units) *compute_units = ctx().compute_units;
    if (clock_khz) *clock_khz = ctx().clock_khz;
    return MNI_OK;
}

int mni_rocm_device_xcds(void) {
    MNI_API_GUARD;
    if (ensure_init() != MNI_OK) return -1;
    return ctx().xcd_count;
}

const char *mni_rocm_last_error(void) { return g_err_shared; }

int mni_rocm_malloc(void **ptr, size_t bytes) {
    MNI_API_GUARD;
    if (!ptr) return set_error(MNI_ERR_INVALID, "null out pointer");
    return dev_alloc(ptr, bytes);
}
int mni_rocm_free(void *ptr) { MNI_API_GUARD; return dev_free(ptr); }
int mni_rocm_clear_cache(void) { MNI_API_GUARD; return dev_clear_cache(); }

int mni_rocm_h2d(void *dst, const void *src, size_t bytes) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    if (bytes == 0) return MNI_OK;
    MNI_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx().stream));
    return sync_stream_checked("h2d");
}
int mni_rocm_d2h(void *dst, const void *src, size_t bytes) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    if (bytes == 0) return MNI_OK;
    DeviceCtx &c = ctx();
    if (bytes <= DeviceCtx::STAGE_BYTES && bytes % 4 == 0 && ((uintptr_t)src & 3) == 0 && c.fetch_host) {
        // a small read (a loss, a norm, a few hundred values): a kernel brings it to pinned host memory and
        // says so; no copy to set up, no barrier to wait behind
        const unsigned tag = next_result_tag();
        hipLaunchKernelGGL(fetch_small_kernel, dim3(1), dim3(256), 0, c.stream, c.fetch_dev, (const unsigned *)src, (int)(bytes / 4),
                           c.result_dev, tag);
        MNI_TRY(check_launch("fetch_small_kernel"));
        int rc = MNI_OK;
        if (poll_result_word(tag, nullptr, 150)) rc = check_device_status("d2h");
        else rc = blocking_sync("d2h");
        if (rc == MNI_OK) memcpy(dst, c.fetch_host, bytes);
        return rc;
    }
    MNI_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, c.stream));
    return sync_stream_checked("d2h");
}
int mni_rocm_d2d(void *dst, const void *src, size_t bytes) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    if (bytes == 0) return MNI_OK;
    MNI_HIP_CHECK(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx().stream));
    return MNI_OK;
}
int mni_rocm_sync(void) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    return sync_stream_checked("sync");
}

int mni_rocm_sgemm_noalloc(const mni_gemm_desc *desc) {
    MNI_API_GUARD;
    if (!desc) return set_error(MNI_ERR_INVALID, "sgemm_noalloc: null descriptor");
    DeviceCtx &c = ctx();
    // Initialisation allocates (stream, flag array); this call must not, so it does not initialise.
    if (!c.ready || !c.noalloc_scratch)
        return set_error(MNI_ERR_INVALID, "sgemm_noalloc: call mni_rocm_init first (this entry point allocates nothing, "
                                          "initialisation does)");
    c.scratch = c.noalloc_scratch;
    c.scratch_bytes = c.noalloc_scratch_bytes;
    const int rc = sgemm(*desc);
    c.scratch = nullptr;
    c.scratch_bytes = 0;
    return rc;
}

size_t mni_rocm_sgemm_noalloc_workspace_bytes(void) { return NOALLOC_SCRATCH_BYTES; }

uint64_t mni_rocm_launch_count(void) {
    MNI_API_GUARD;
    return ctx().launches;
}

int mni_rocm_alloc_stats(uint64_t *requests, uint64_t *driver_allocations, uint64_t *releases, uint64_t *cached_bytes) {
    MNI_API_GUARD;
    if (!requests || !driver_allocations || !releases || !cached_bytes) return set_error(MNI_ERR_INVALID, "alloc_stats: null output");
    dev_alloc_stats(requests, driver_allocations, releases, cached_bytes);
    return MNI_OK;
}

int mni_rocm_test_raise_device_status(unsigned code) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    *(volatile unsigned *)ctx().status_host = code;
    return MNI_OK;
}

int mni_rocm_event_create(void **event) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    if (!event) return set_error(MNI_ERR_INVALID, "null out pointer");
    hipEvent_t e;
    MNI_HIP_CHECK(hipEventCreate(&e));
    *event = (void *)e;
    return MNI_OK;
}
int mni_rocm_event_record(void *event) {
    MNI_API_GUARD;
    MNI_TRY(ensure_init());
    MNI_HIP_CHECK(hipEventRecord((hipEvent_t)event, ctx().stream));
    return MNI_OK;
}
int mni_rocm_event_elapsed_ms(void *start, void *stop, float *ms) {
    MNI_API_GUARD;
    MNI_HIP_CHECK(hipEventSynchronize((hipEvent_t)stop));
    MNI_HIP_CHECK(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
    return check_device_status("event_elapsed_ms");
}
int mni_rocm_event_destroy(void *event) {
    MNI_API_GUARD;
    MNI_HIP_CHECK(hipEventDestroy((hipEvent_t)event));
    return MNI_OK;
}

}  // extern "C"
