// runtime.hip -- library state, streams, copies and the allocator's device backend.
//
// Replaces zenu-cuda/src/lib.rs:18-25,60-72 (process-global state) and
// zenu-cuda/src/runtime/mod.rs (cudaMallocAsync + synchronise, blocking memcpy, stream and
// mem-pool setup) for the HIP device.
#include <stdlib.h>
#include <string.h>

#include <mutex>

#include "allocator.hpp"
#include "common.hpp"

namespace zenu {

static thread_local hipError_t tl_last_hip_error = hipSuccess;
void set_last_hip_error(hipError_t e) { tl_last_hip_error = e; }

namespace {

struct HipBackend : AllocBackend {
    int raw_alloc(void **p, size_t bytes) override
    {
        hipError_t e = hipMalloc(p, bytes);
        if (e != hipSuccess) {
            (void)hipGetLastError();  // clear the sticky out-of-memory error
            *p = nullptr;
            return 1;
        }
        return 0;
    }
    int raw_free(void *p) override { return hipFree(p) == hipSuccess ? 0 : 1; }
    int order_after(void *owner, void *waiter) override
    {
        hipEvent_t ev;
        if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) return 1;
        int rc = 0;
        if (hipEventRecord(ev, static_cast<hipStream_t>(owner)) != hipSuccess) rc = 1;
        if (!rc && hipStreamWaitEvent(static_cast<hipStream_t>(waiter), ev, 0) != hipSuccess) rc = 1;
        (void)hipEventDestroy(ev);  // released by the runtime once the record has completed
        return rc;
    }
    int device_synchronize() override { return hipDeviceSynchronize() == hipSuccess ? 0 : 1; }
};

constexpr int64_t kNumCounters = 1 << 16;

struct State {
    bool ready = false;
    bool use_pool = true;
    int *counters = nullptr;      // arrival counters of the reductions, zero at rest
    int64_t counter_cursor = 0;
    std::mutex counter_mu;
    DeviceInfo info;
    HipBackend backend;
    CachingAllocator *pool = nullptr;
};

State g_state;
std::mutex g_init_mu;

int init_locked(int device)
{
    if (g_state.ready) {
        if (device == g_state.info.device) return ZENU_OK;
        return ZENU_ERR_ARG;  // one device per process, as the reference (device 0 hard-coded)
    }
    int count = 0;
    ZENU_HIP_TRY(hipGetDeviceCount(&count));
    if (device < 0 || device >= count) return ZENU_ERR_ARG;
    ZENU_HIP_TRY(hipSetDevice(device));
    hipDeviceProp_t prop;
    ZENU_HIP_TRY(hipGetDeviceProperties(&prop, device));
    g_state.info.device = device;
    g_state.info.num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    g_state.info.lds_per_block = prop.sharedMemPerBlock;
    const char *env = getenv("ZENU_USE_MEMPOOL");  // zenu-matrix/src/lib.rs:36, default "1"
    g_state.use_pool = !(env && strcmp(env, "0") == 0);
    g_state.pool = new CachingAllocator(&g_state.backend);
    ZENU_HIP_TRY(hipMalloc(reinterpret_cast<void **>(&g_state.counters), kNumCounters * sizeof(int)));
    ZENU_HIP_TRY(hipMemset(g_state.counters, 0, kNumCounters * sizeof(int)));
    g_state.counter_cursor = 0;
    g_state.ready = true;
    return ZENU_OK;
}

__global__ void fill_zero_kernel(uint4 *dst16, size_t n16, unsigned char *tail, size_t ntail)
{
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t step = (size_t)gridDim.x * blockDim.x;
    for (size_t k = i; k < n16; k += step) dst16[k] = make_uint4(0, 0, 0, 0);
    if (i < ntail) tail[i] = 0;
}

}  // namespace

const DeviceInfo &device_info() { return g_state.info; }

// Consecutive launches take consecutive ranges of the ring, so a range is reused only after
// kNumCounters counters' worth of later reductions; every kernel leaves its counters at zero.
int *reserve_counters(int64_t n)
{
    if (n <= 0 || n > kNumCounters || !g_state.counters) return nullptr;
    std::lock_guard<std::mutex> g(g_state.counter_mu);
    if (g_state.counter_cursor + n > kNumCounters) g_state.counter_cursor = 0;
    int *r = g_state.counters + g_state.counter_cursor;
    g_state.counter_cursor += n;
    return r;
}

int ensure_init()
{
    if (g_state.ready) return ZENU_OK;
    std::lock_guard<std::mutex> g(g_init_mu);
    return init_locked(0);
}

Workspace::Workspace(size_t bytes, hipStream_t s) : stream(s)
{
    if (bytes) status = zenu_hip_malloc(&ptr, bytes, s);
}
Workspace::~Workspace()
{
    if (ptr) zenu_hip_free(ptr, stream);
}

}  // namespace zenu

using namespace zenu;

extern "C" {

int zenu_hip_init(int device)
{
    std::lock_guard<std::mutex> g(g_init_mu);
    return init_locked(device);
}

int zenu_hip_shutdown(void)
{
    std::lock_guard<std::mutex> g(g_init_mu);
    if (!g_state.ready) return ZENU_OK;
    (void)hipDeviceSynchronize();
    delete g_state.pool;
    g_state.pool = nullptr;
    if (g_state.counters) (void)hipFree(g_state.counters);
    g_state.counters = nullptr;
    g_state.ready = false;
    return ZENU_OK;
}

const char *zenu_hip_status_string(int status)
{
    switch (status) {
    case ZENU_OK: return "ok";
    case ZENU_ERR_RANK: return "The rank of the matrix is different.";
    case ZENU_ERR_SHAPE: return "shape mismatch / shapes are not broadcast compatible";
    case ZENU_ERR_AXIS: return "Invalid axis";
    case ZENU_ERR_ARG: return "invalid argument";
    case ZENU_ERR_HIP: return "HIP runtime error";
    case ZENU_ERR_OOM: return "out of device memory";
    case ZENU_ERR_UNSUPPORTED: return "unsupported";
    case ZENU_ERR_NOT_OWNED: return "pointer not owned by the memory pool";
    default: return "unknown status";
    }
}

int zenu_hip_last_hip_error(void) { return (int)tl_last_hip_error; }
const char *zenu_hip_last_hip_error_string(void) { return hipGetErrorString(tl_last_hip_error); }

int zenu_hip_stream_create(zenu_stream_t *stream)
{
    if (!stream) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s;
    // default flags and priority: ordered against the null stream, as the reference's
    // cudaStreamCreate stream is (zenu-cuda/src/runtime/mod.rs:113-121)
    ZENU_HIP_TRY(hipStreamCreate(&s));
    *stream = s;
    return ZENU_OK;
}

int zenu_hip_stream_destroy(zenu_stream_t stream)
{
    if (!stream) return ZENU_ERR_ARG;
    ZENU_HIP_TRY(hipStreamDestroy(as_stream(stream)));
    return ZENU_OK;
}

int zenu_hip_stream_synchronize(zenu_stream_t stream)
{
    ZENU_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return ZENU_OK;
}

int zenu_hip_device_synchronize(void)
{
    ZENU_HIP_TRY(hipDeviceSynchronize());
    return ZENU_OK;
}

int zenu_hip_malloc(void **ptr_dev, size_t bytes, zenu_stream_t stream)
{
    if (!ptr_dev) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    if (!g_state.use_pool) {
        *ptr_dev = nullptr;
        if (g_state.backend.raw_alloc(ptr_dev, bytes ? bytes : 1) != 0) return ZENU_ERR_OOM;
        return ZENU_OK;
    }
    return g_state.pool->malloc(ptr_dev, bytes, stream);
}

int zenu_hip_free(void *ptr_dev, zenu_stream_t stream)
{
    if (!ptr_dev) return ZENU_OK;
    int rc = ensure_init();
    if (rc) return rc;
    if (!g_state.use_pool) {
        ZENU_HIP_TRY(hipFree(ptr_dev));
        return ZENU_OK;
    }
    return g_state.pool->free(ptr_dev, stream);
}

int zenu_hip_mempool_trim(void)
{
    int rc = ensure_init();
    if (rc) return rc;
    return g_state.pool->trim();
}

int zenu_hip_mempool_stats(zenu_mempool_stats_t *out)
{
    if (!out) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    AllocStats s = g_state.pool->stats();
    out->bytes_in_use = s.bytes_in_use;
    out->bytes_cached = s.bytes_cached;
    out->bytes_reserved = s.bytes_reserved;
    out->n_alloc_calls = s.n_alloc_calls;
    out->n_cache_hits = s.n_cache_hits;
    out->n_driver_allocs = s.n_driver_allocs;
    out->n_driver_frees = s.n_driver_frees;
    out->n_oom_retries = s.n_oom_retries;
    return ZENU_OK;
}

int zenu_hip_raw_malloc(void **ptr_dev, size_t bytes)
{
    if (!ptr_dev) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    if (g_state.backend.raw_alloc(ptr_dev, bytes ? bytes : 1) != 0) return ZENU_ERR_OOM;
    return ZENU_OK;
}

int zenu_hip_raw_free(void *ptr_dev)
{
    if (!ptr_dev) return ZENU_OK;
    ZENU_HIP_TRY(hipFree(ptr_dev));
    return ZENU_OK;
}

int zenu_hip_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, zenu_stream_t stream)
{
    if (bytes == 0) return ZENU_OK;
    if (!dst_dev || !src_host) return ZENU_ERR_ARG;
    ZENU_HIP_TRY(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, as_stream(stream)));
    ZENU_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return ZENU_OK;
}

int zenu_hip_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, zenu_stream_t stream)
{
    if (bytes == 0) return ZENU_OK;
    if (!dst_host || !src_dev) return ZENU_ERR_ARG;
    ZENU_HIP_TRY(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, as_stream(stream)));
    ZENU_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
    return ZENU_OK;
}

int zenu_hip_memcpy_d2d(void *dst_dev, const void *src_dev, size_t bytes, zenu_stream_t stream)
{
    if (bytes == 0) return ZENU_OK;
    if (!dst_dev || !src_dev) return ZENU_ERR_ARG;
    ZENU_HIP_TRY(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
    return ZENU_OK;
}

int zenu_hip_memset_zero(void *dst_dev, size_t bytes, zenu_stream_t stream)
{
    if (bytes == 0) return ZENU_OK;
    if (!dst_dev) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    // a fill kernel rather than hipMemsetAsync, so the call can sit inside a captured graph
    uintptr_t a = reinterpret_cast<uintptr_t>(dst_dev);
    size_t head = (16 - (a & 15)) & 15;
    if (head > bytes) head = bytes;
    unsigned char *p = static_cast<unsigned char *>(dst_dev);
    size_t n16 = (bytes - head) / 16;
    size_t tail = bytes - head - n16 * 16;
    if (head) {
        fill_zero_kernel<<<1, 64, 0, as_stream(stream)>>>(nullptr, 0, p, head);
        ZENU_LAUNCH_CHECK();
    }
    if (n16 || tail) {
        size_t want = (n16 + 255) / 256;
        unsigned grid = (unsigned)(want < 1 ? 1 : (want > 4096 ? 4096 : want));
        fill_zero_kernel<<<grid, 256, 0, as_stream(stream)>>>(
            reinterpret_cast<uint4 *>(p + head), n16, p + head + n16 * 16, tail);
        ZENU_LAUNCH_CHECK();
    }
    return ZENU_OK;
}

}  // extern "C"
