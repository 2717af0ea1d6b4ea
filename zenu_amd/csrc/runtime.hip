// runtime.hip -- library state, streams, copies and the allocator's device backend.
//
// Replaces zenu-cuda/src/lib.rs:18-25,60-72 (process-global state) and
// zenu-cuda/src/runtime/mod.rs (cudaMallocAsync + synchronise, blocking memcpy, stream and
// mem-pool setup) for the HIP device.
#include <stdlib.h>
#include <string.h>

#include <atomic>
#include <map>
#include <mutex>

#include "allocator.hpp"
#include "common.hpp"

namespace zenu {

int init_static_scratch();   // reduce.hip

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
constexpr int64_t kNumSlotWords = 1 << 19;       // 4 MiB of tagged 64-bit partial-result words per stream
constexpr size_t kRingBytes = kNumCounters * sizeof(int) + kNumSlotWords * sizeof(uint64_t);

struct State {
    std::atomic<bool> ready{false};   // read without the init lock by every entry point
    bool use_pool = true;
    // cross-workgroup memory of the split reductions, one ring per stream, because only launches on
    // the same stream are certain to run one after the other: arrival counters (zero at rest), then
    // tagged partial-result words.  A word is {tag, payload}; the tag is the ring's launch number
    // (`epoch`, never zero, never repeated), so what an earlier launch left behind is never taken
    // for a result of the current one and nothing has to be cleared.
    struct Ring { int *base = nullptr; int64_t cursor = 0; int64_t slot_cursor = 0; uint32_t epoch = 0; size_t rehearsed = 0; };
    std::map<hipStream_t, Ring> rings;
    std::mutex counter_mu;
    DeviceInfo info;
    HipBackend backend;
    CachingAllocator *pool = nullptr;
};

State g_state;
std::mutex g_init_mu;
// polls (about a microsecond each) before a folding workgroup computes missing partials itself:
// about as long as recomputing every split of a 128 MiB reduction takes one workgroup (6 ms at
// 22 GB/s); waiting longer than that for workgroups that have not been dispatched buys nothing
std::atomic<int> g_reduce_spin_limit{1 << 13};

// is `stream` recording a graph?  (the null stream never is)
bool stream_is_capturing(hipStream_t stream)
{
    if (!stream) return false;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    return st != hipStreamCaptureStatusNone;
}

// allocate and clear the ring of `stream` (blocking; at init, at stream creation, or at the first
// split reduction on a stream the library did not create).  Not while that stream records a
// graph: the blocking calls would invalidate the capture.
int *make_ring(hipStream_t stream)
{
    if (stream_is_capturing(stream)) return nullptr;
    int *base = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&base), kRingBytes);
    if (e == hipSuccess) e = hipMemset(base, 0, kRingBytes);
    if (e == hipSuccess) e = hipDeviceSynchronize();
    if (e != hipSuccess) {
        set_last_hip_error(e);
        if (base) (void)hipFree(base);
        return nullptr;
    }
    std::lock_guard<std::mutex> g(g_state.counter_mu);
    State::Ring &r = g_state.rings[stream];
    if (r.base) {           // another thread was faster
        (void)hipFree(base);
        return r.base;
    }
    r.base = base;
    r.cursor = 0;
    return base;
}

void drop_ring(hipStream_t stream)
{
    std::lock_guard<std::mutex> g(g_state.counter_mu);
    auto it = g_state.rings.find(stream);
    if (it == g_state.rings.end()) return;
    if (it->second.base) (void)hipFree(it->second.base);
    g_state.rings.erase(it);
}

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
    int rc = init_static_scratch();
    if (rc) return rc;
    g_state.pool = new CachingAllocator(&g_state.backend);
    g_state.ready = true;
    return make_ring(nullptr) ? ZENU_OK : ZENU_ERR_HIP;   // the null stream's ring; created streams get theirs at creation
}

// each workgroup clears 8 KiB (256 threads x two 16-byte stores); many short workgroups stream
// stores faster than a capped grid of looping ones (46.9 us against 60.7 us for 256 MiB)
constexpr int kFillBlock = 256, kFillUnroll = 2;
__global__ __launch_bounds__(kFillBlock) void fill_zero_kernel(uint4 *dst16, size_t n16, unsigned char *tail, size_t ntail)
{
    const size_t base = (size_t)blockIdx.x * (kFillBlock * kFillUnroll) + threadIdx.x;
#pragma unroll
    for (int u = 0; u < kFillUnroll; u++) {
        const size_t k = base + (size_t)u * kFillBlock;
        if (k < n16) dst16[k] = make_uint4(0, 0, 0, 0);
    }
    if (blockIdx.x == 0 && threadIdx.x < ntail) tail[threadIdx.x] = 0;
}

}  // namespace

const DeviceInfo &device_info() { return g_state.info; }
bool library_ready() { return g_state.ready; }
int reduce_spin_limit() { return g_reduce_spin_limit.load(std::memory_order_relaxed); }

// Consecutive launches on a stream take consecutive ranges of that stream's ring; a range is reused
// by a later launch of the same stream, which runs after the earlier one.  Every kernel leaves
// its counters at zero.
int *reserve_counters(int64_t n, hipStream_t stream)
{
    if (n <= 0 || n > kNumCounters || !g_state.ready) return nullptr;
    {
        std::lock_guard<std::mutex> g(g_state.counter_mu);
        auto it = g_state.rings.find(stream);
        if (it != g_state.rings.end() && it->second.base) {
            State::Ring &r = it->second;
            if (r.cursor + n > kNumCounters) r.cursor = 0;
            int *out = r.base + r.cursor;
            r.cursor += n;
            return out;
        }
    }
    if (!make_ring(stream)) return nullptr;
    return reserve_counters(n, stream);
}

// `nwords` consecutive tagged words from the ring of `stream` and the tag (`*epoch`) that marks
// this launch's results, or nullptr: the request is larger than half the ring, the stream has no
// ring and cannot get one now, or the stream is recording a graph (a recorded launch would replay
// its tag; such launches use the counters instead).
uint64_t *reserve_slots(int64_t nwords, hipStream_t stream, uint32_t *epoch)
{
    if (nwords <= 0 || nwords > kNumSlotWords / 2 || !g_state.ready) return nullptr;
    if (stream_is_capturing(stream)) return nullptr;
    for (int attempt = 0; attempt < 2; attempt++) {
        {
            std::lock_guard<std::mutex> g(g_state.counter_mu);
            auto it = g_state.rings.find(stream);
            if (it != g_state.rings.end() && it->second.base) {
                State::Ring &r = it->second;
                if (r.epoch == 0xffffffffu) {
                    // every tag has been used once: start over on a cleared ring (once in 2^32 launches)
                    if (hipStreamSynchronize(stream) != hipSuccess) return nullptr;
                    if (hipMemset(r.base + kNumCounters, 0, kNumSlotWords * sizeof(uint64_t)) != hipSuccess) return nullptr;
                    if (hipDeviceSynchronize() != hipSuccess) return nullptr;
                    r.epoch = 0;
                }
                if (r.slot_cursor + nwords > kNumSlotWords) r.slot_cursor = 0;
                uint64_t *out = reinterpret_cast<uint64_t *>(r.base + kNumCounters) + r.slot_cursor;
                r.slot_cursor += nwords;
                *epoch = ++r.epoch;
                return out;
            }
        }
        if (!make_ring(stream)) return nullptr;
    }
    return nullptr;
}

// A split reduction that uses tagged words needs no workspace, but the same call recorded into a
// graph would (it takes the counter path): the eager call then requests and releases a block of
// that size once, so the pool of its stream holds one when a capture comes.  True when `bytes` is
// larger than anything rehearsed on `stream` so far; never with the pool switched off (the block
// would go straight back to the driver).
bool rehearsal_needed(size_t bytes, hipStream_t stream)
{
    if (!g_state.use_pool || bytes == 0) return false;
    std::lock_guard<std::mutex> g(g_state.counter_mu);
    auto it = g_state.rings.find(stream);
    if (it == g_state.rings.end()) return false;
    if (bytes <= it->second.rehearsed) return false;
    it->second.rehearsed = bytes;
    return true;
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
    {
        std::lock_guard<std::mutex> gc(g_state.counter_mu);
        for (auto &kv : g_state.rings)
            if (kv.second.base) (void)hipFree(kv.second.base);
        g_state.rings.clear();
    }
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
    case ZENU_ERR_NOT_INIT: return "zenu_hip_init has not run (this entry point may not initialise the library: that allocates)";
    case ZENU_ERR_SCRATCH_LIMIT: return "request needs more than the static scratch of the allocation-free entry point";
    default: return "unknown status";
    }
}

const char *zenu_hip_validated_libm(void)
{
    return "glibc 2.35 libm, x86-64 (the variants selected on CPUs with FMA)";
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
    if (!make_ring(s)) {
        (void)hipStreamDestroy(s);
        return ZENU_ERR_HIP;
    }
    if (g_state.pool) g_state.pool->adopt_stream(s);
    *stream = s;
    return ZENU_OK;
}

int zenu_hip_stream_destroy(zenu_stream_t stream)
{
    if (!stream) return ZENU_ERR_ARG;
    ZENU_HIP_TRY(hipStreamSynchronize(as_stream(stream)));   // its reductions are done with their counters
    drop_ring(as_stream(stream));
    if (g_state.pool) g_state.pool->retire_stream(stream);   // its cached blocks outlive it
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
        // Without the pool every request goes to the driver and every release is a hipFree, which
        // synchronises: inside a capture that invalidates the recording or, in relaxed mode, frees
        // memory whose address the recorded kernels keep.  Refused before anything is recorded.
        if (stream_is_capturing(as_stream(stream))) return ZENU_ERR_UNSUPPORTED;
        *ptr_dev = nullptr;
        if (g_state.backend.raw_alloc(ptr_dev, bytes ? bytes : 1) != 0) return ZENU_ERR_OOM;
        return ZENU_OK;
    }
    return g_state.pool->malloc(ptr_dev, bytes, stream, stream_is_capturing(as_stream(stream)));
}

int zenu_hip_free(void *ptr_dev, zenu_stream_t stream)
{
    if (!ptr_dev) return ZENU_OK;
    int rc = ensure_init();
    if (rc) return rc;
    if (!g_state.use_pool) {
        if (stream_is_capturing(as_stream(stream))) return ZENU_ERR_UNSUPPORTED;   // see zenu_hip_malloc
        ZENU_HIP_TRY(hipFree(ptr_dev));
        return ZENU_OK;
    }
    return g_state.pool->free(ptr_dev, stream);
}

int zenu_hip_set_reduce_spin_limit(int polls)
{
    if (polls < 0) return ZENU_ERR_ARG;
    g_reduce_spin_limit.store(polls, std::memory_order_relaxed);
    return ZENU_OK;
}

int zenu_hip_release_captured(zenu_stream_t stream)
{
    int rc = ensure_init();
    if (rc) return rc;
    if (stream_is_capturing(as_stream(stream))) return ZENU_ERR_ARG;
    if (g_state.pool) g_state.pool->release_captured(stream);
    return ZENU_OK;
}

int zenu_hip_mempool_trim(void)
{
    int rc = ensure_init();
    if (rc) return rc;
    {   // the blocks that rehearsals left are gone with the rest
        std::lock_guard<std::mutex> g(g_state.counter_mu);
        for (auto &kv : g_state.rings) kv.second.rehearsed = 0;
    }
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
        fill_zero_kernel<<<1, kFillBlock, 0, as_stream(stream)>>>(nullptr, 0, p, head);
        ZENU_LAUNCH_CHECK();
    }
    if (n16 || tail) {
        const size_t per_block = (size_t)kFillBlock * kFillUnroll;
        const size_t want = (n16 + per_block - 1) / per_block;
        if (want > 0x7fffffffull) return ZENU_ERR_UNSUPPORTED;
        const unsigned grid = (unsigned)(want < 1 ? 1 : want);
        fill_zero_kernel<<<grid, kFillBlock, 0, as_stream(stream)>>>(
            reinterpret_cast<uint4 *>(p + head), n16, p + head + n16 * 16, tail);
        ZENU_LAUNCH_CHECK();
    }
    return ZENU_OK;
}

}  // extern "C"
