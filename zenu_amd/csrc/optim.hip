// optim.hip -- fused SGD / Adam / AdamW parameter updates for gfx950.
//
// The reference composes each update from Matrix operators: about 14 launches, 9 temporaries and
// 33 f32 streams per element for Adam (zenu-optimizer/src/adam.rs:44-56), two launches for SGD
// (zenu-optimizer/src/sgd.rs:23-27).  Here one launch reads p, g, m, v and writes p, m, v:
// 7 streams, 28 B per f32 parameter, 128-bit accesses, HBM bound.
//
// The per-element arithmetic is the reference's operator chain with a rounding to T after every
// step (contraction is off, / and sqrt are the correctly rounded IEEE ones), so results are
// bit-identical to the CPU path:
//   m1 = m*b1; t = g*(1-b1); m2 = m1+t
//   v1 = v*b2; q = g*g; u = q*(1-b2); v2 = v1+u
//   mh = m2/(1-b1^t); vh = v2/(1-b2^t); d = sqrt(vh)+eps; upd = mh/d
//   [AdamW, weights only] p = p - (p*lr)*wd          (zenu-optimizer/src/adamw.rs:61-65)
//   p = p - upd*lr
// 1-b, b^t and 1-b^t are formed on the host in T, as adam.rs:22-25,45-51 does.
#include <math.h>

#include <vector>

#include "common.hpp"
#include "vecmem.hpp"

namespace zenu {
namespace {

#ifndef ZENU_ADAM_BLOCK
#define ZENU_ADAM_BLOCK 128
#endif
#ifndef ZENU_ADAM_UNROLL
#define ZENU_ADAM_UNROLL 2
#endif
constexpr int kBlock = ZENU_ADAM_BLOCK;   // small workgroups measured best for the 7-stream update (6.2 vs 5.9 TB/s at 256)
constexpr int kUnroll = ZENU_ADAM_UNROLL;


template <typename T> struct AdamConsts {
    T lr, beta1, beta2, eps, omb1, omb2, c1, c2, wd;
};

template <typename T>
__device__ __forceinline__ void adam_elem(T &p, T g, T &m, T &v, const AdamConsts<T> &k, bool decay)
{
    T m1 = m * k.beta1;
    T t = g * k.omb1;
    T m2 = m1 + t;
    T v1 = v * k.beta2;
    T q = g * g;
    T u = q * k.omb2;
    T v2 = v1 + u;
    T mh = m2 / k.c1;
    T vh = v2 / k.c2;
    T d = sqrt(vh) + k.eps;
    T upd = mh / d;
    T pp = p;
    if (decay) {
        T w = pp * k.lr;
        w = w * k.wd;
        pp = pp - w;
    }
    T s = upd * k.lr;
    p = pp - s;
    m = m2;
    v = v2;
}

template <typename T, int VEC, bool NT>
__device__ __forceinline__ void adam_tile(T *p, const T *g, T *m, T *v, int64_t base, int tid,
                                          const AdamConsts<T> &k, bool decay)
{
    Pack<T, VEC> vp[kUnroll], vg[kUnroll], vm[kUnroll], vv[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const int64_t i = base + ((int64_t)u * kBlock + tid) * VEC;
        vp[u] = load_pack<T, VEC, NT>(p + i);
        vg[u] = load_pack<T, VEC, NT>(g + i);
        vm[u] = load_pack<T, VEC, NT>(m + i);
        vv[u] = load_pack<T, VEC, NT>(v + i);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const int64_t i = base + ((int64_t)u * kBlock + tid) * VEC;
#pragma unroll
        for (int j = 0; j < VEC; j++) adam_elem<T>(vp[u].v[j], vg[u].v[j], vm[u].v[j], vv[u].v[j], k, decay);
        store_pack<T, VEC, NT>(p + i, vp[u]);
        store_pack<T, VEC, NT>(m + i, vm[u]);
        store_pack<T, VEC, NT>(v + i, vv[u]);
    }
}

// one tile of kBlock * VEC * kUnroll elements.  NT (stream the tensors) is a template parameter:
// a run-time `if (nt) load_nt else load` is merged by the compiler into one plain load.
template <typename T, int VEC, bool NT>
__device__ __forceinline__ void adam_span(T *p, const T *g, T *m, T *v, int64_t n, int64_t blk,
                                          const AdamConsts<T> &k, bool decay)
{
    constexpr int64_t kTile = (int64_t)kBlock * VEC * kUnroll;
    const int64_t base = blk * kTile;
    const int tid = threadIdx.x;
    if (VEC > 1 && base + kTile <= n) {
        adam_tile<T, VEC, NT>(p, g, m, v, base, tid, k, decay);
    } else {
        for (int u = 0; u < kUnroll; u++) {
            const int64_t i0 = base + ((int64_t)u * kBlock + tid) * VEC;
            for (int j = 0; j < VEC; j++) {
                const int64_t i = i0 + j;
                if (i < n) {
                    T pe = p[i], me = m[i], ve = v[i];
                    adam_elem<T>(pe, g[i], me, ve, k, decay);
                    p[i] = pe;
                    m[i] = me;
                    v[i] = ve;
                }
            }
        }
    }
}

template <typename T, int VEC, bool NT>
__global__ __launch_bounds__(kBlock) void adam_kernel(T *p, const T *g, T *m, T *v, int64_t n,
                                                      AdamConsts<T> k, int decay)
{
    adam_span<T, VEC, NT>(p, g, m, v, n, blockIdx.x, k, decay != 0);
}

// multi-tensor: up to kMaxMulti tensors per launch, described in the kernel arguments themselves
// (no staging buffer, no copy, nothing to synchronise; the call can sit in a captured graph).
// first_block[i] is the first workgroup of tensor i; a workgroup finds its tensor by a short scan.
constexpr int kMaxMulti = 24;
struct MultiEntry {
    void *p;
    const void *g;
    void *m;
    void *v;
    int64_t n;
    int32_t decay;
    int32_t vec_ok;
};
struct MultiArgs {
    MultiEntry e[kMaxMulti];
    int32_t first_block[kMaxMulti + 1];
    int32_t count;
};

// The step-dependent scalars of a scheduled update: 1 - beta1^t and 1 - beta2^t for consecutive
// steps t, formed on the host in T exactly as an eager call forms them, and a cursor on the device
// that says which pair the next update uses.  A launch recorded into a graph carries the schedule's
// address, not a step number, so every replay is the next step.
struct ScheduleHeader {
    uint32_t cursor;      // index of the pair the next update uses
    uint32_t n;           // pairs in the table
    uint32_t exhausted;   // updates that were asked for after the last pair (they change nothing)
    uint32_t pad;
};

template <typename T>
__device__ __forceinline__ bool schedule_consts(const ScheduleHeader *h, AdamConsts<T> &k)
{
    if (!h) return true;
    const uint32_t i = h->cursor;
    if (i >= h->n) return false;
    const T *table = reinterpret_cast<const T *>(h + 1);
    k.c1 = table[2 * i];
    k.c2 = table[2 * i + 1];
    return true;
}

// after every launch of one scheduled update: move on to the next step
__global__ void schedule_advance_kernel(ScheduleHeader *h)
{
    if (h->cursor < h->n) h->cursor = h->cursor + 1;
    else h->exhausted = h->exhausted + 1;
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void adam_multi_kernel(MultiArgs a, AdamConsts<T> k, const ScheduleHeader *sched)
{
    if (!schedule_consts<T>(sched, k)) return;
    int t = 0;
    while (t + 1 < a.count && (int)blockIdx.x >= a.first_block[t + 1]) t++;
    const MultiEntry &e = a.e[t];
    const int64_t tile = (int64_t)blockIdx.x - a.first_block[t];
    T *p = static_cast<T *>(e.p);
    const T *g = static_cast<const T *>(e.g);
    T *m = static_cast<T *>(e.m);
    T *v = static_cast<T *>(e.v);
    if (e.vec_ok) adam_span<T, VEC, false>(p, g, m, v, e.n, tile, k, e.decay != 0);
    else {
        // unaligned tensor: same tile, scalar accesses
        constexpr int64_t kTile = (int64_t)kBlock * VEC * kUnroll;
        const int64_t base = tile * kTile;
        for (int64_t i = base + threadIdx.x; i < base + kTile && i < e.n; i += kBlock) {
            T pe = p[i], me = m[i], ve = v[i];
            adam_elem<T>(pe, g[i], me, ve, k, e.decay != 0);
            p[i] = pe;
            m[i] = me;
            v[i] = ve;
        }
    }
}

constexpr int kSgdUnroll = 4;

// one tile of kBlock * VEC * kSgdUnroll elements: p = p - (g * lr), two roundings (sgd.rs:23-27)
template <typename T, int VEC>
__device__ __forceinline__ void sgd_span(T *p, const T *g, int64_t n, int64_t blk, T lr)
{
    constexpr int kU = kSgdUnroll;
    constexpr int64_t kTile = (int64_t)kBlock * VEC * kU;
    const int64_t base = blk * kTile;
    const int tid = threadIdx.x;
    if (VEC > 1 && base + kTile <= n) {
        Pack<T, VEC> vp[kU], vg[kU];
#pragma unroll
        for (int u = 0; u < kU; u++) {
            const int64_t i = base + ((int64_t)u * kBlock + tid) * VEC;
            vp[u] = load_pack<T, VEC, true>(p + i);
            vg[u] = load_pack<T, VEC, true>(g + i);
        }
#pragma unroll
        for (int u = 0; u < kU; u++) {
            const int64_t i = base + ((int64_t)u * kBlock + tid) * VEC;
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                T t = vg[u].v[j] * lr;          // sgd.rs:24
                vp[u].v[j] = vp[u].v[j] - t;    // sgd.rs:27
            }
            store_pack<T, VEC, true>(p + i, vp[u]);
        }
    } else {
        for (int u = 0; u < kU; u++) {
            const int64_t i0 = base + ((int64_t)u * kBlock + tid) * VEC;
            for (int j = 0; j < VEC; j++) {
                const int64_t i = i0 + j;
                if (i < n) {
                    T t = g[i] * lr;
                    p[i] = p[i] - t;
                }
            }
        }
    }
}

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void sgd_kernel(T *p, const T *g, int64_t n, T lr)
{
    sgd_span<T, VEC>(p, g, n, blockIdx.x, lr);
}

// multi-tensor SGD: the tensors of one SGD::update (sgd.rs:20-31 walks the parameter map) in one
// launch; same argument layout as the multi-tensor Adam (m, v unused)
template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void sgd_multi_kernel(MultiArgs a, T lr)
{
    int t = 0;
    while (t + 1 < a.count && (int)blockIdx.x >= a.first_block[t + 1]) t++;
    const MultiEntry &e = a.e[t];
    const int64_t tile = (int64_t)blockIdx.x - a.first_block[t];
    T *p = static_cast<T *>(e.p);
    const T *g = static_cast<const T *>(e.g);
    if (e.vec_ok) sgd_span<T, VEC>(p, g, e.n, tile, lr);
    else {
        constexpr int64_t kTile = (int64_t)kBlock * VEC * kSgdUnroll;   // same tile, scalar accesses
        const int64_t base = tile * kTile;
        for (int64_t i = base + threadIdx.x; i < base + kTile && i < e.n; i += kBlock) {
            T t2 = g[i] * lr;
            p[i] = p[i] - t2;
        }
    }
}

template <typename T>
AdamConsts<T> make_consts(double lr, double beta1, double beta2, double eps, double wd, double step)
{
    AdamConsts<T> k;
    k.lr = (T)lr;
    k.beta1 = (T)beta1;
    k.beta2 = (T)beta2;
    k.eps = (T)eps;
    k.wd = (T)wd;
    const T st = (T)step;
    // host-side scalars in T, as adam.rs:22-25,45,48,50-51 (powf -> libm powf / pow)
    const T b1t = sizeof(T) == 4 ? (T)powf((float)k.beta1, (float)st) : (T)pow((double)k.beta1, (double)st);
    const T b2t = sizeof(T) == 4 ? (T)powf((float)k.beta2, (float)st) : (T)pow((double)k.beta2, (double)st);
    k.omb1 = (T)1 - k.beta1;
    k.omb2 = (T)1 - k.beta2;
    k.c1 = (T)1 - b1t;
    k.c2 = (T)1 - b2t;
    return k;
}

// the parameter, gradient and moment arrays of one tensor are four different arrays
inline bool adam_arrays_overlap(const void *p, const void *g, const void *m, const void *v, size_t bytes)
{
    return ranges_overlap(p, bytes, g, bytes) || ranges_overlap(p, bytes, m, bytes) || ranges_overlap(p, bytes, v, bytes) ||
           ranges_overlap(g, bytes, m, bytes) || ranges_overlap(g, bytes, v, bytes) || ranges_overlap(m, bytes, v, bytes);
}

template <typename T>
int adam_t(void *p, const void *g, void *m, void *v, int64_t n, const AdamConsts<T> &k, int decay,
           hipStream_t s)
{
    constexpr int VEC = VecOf<T>::N;
    if (n == 0) return ZENU_OK;
    if (adam_arrays_overlap(p, g, m, v, (size_t)n * sizeof(T))) return ZENU_ERR_ARG;
    const bool vec = aligned16(p) && aligned16(g) && aligned16(m) && aligned16(v);
    const bool nt = n * (int64_t)sizeof(T) * 7 >= kStreamBytes;  // 7 passes exceed the caches: stream
    if (vec) {
        const int64_t tile = (int64_t)kBlock * VEC * kUnroll;
        const int64_t grid = (n + tile - 1) / tile;
        if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
        if (nt)
            adam_kernel<T, VEC, true><<<(unsigned)grid, kBlock, 0, s>>>(
                static_cast<T *>(p), static_cast<const T *>(g), static_cast<T *>(m), static_cast<T *>(v), n, k, decay);
        else
            adam_kernel<T, VEC, false><<<(unsigned)grid, kBlock, 0, s>>>(
                static_cast<T *>(p), static_cast<const T *>(g), static_cast<T *>(m), static_cast<T *>(v), n, k, decay);
    } else {
        const int64_t tile = (int64_t)kBlock * kUnroll;
        const int64_t grid = (n + tile - 1) / tile;
        if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
        adam_kernel<T, 1, false><<<(unsigned)grid, kBlock, 0, s>>>(
            static_cast<T *>(p), static_cast<const T *>(g), static_cast<T *>(m), static_cast<T *>(v), n, k, decay);
    }
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

template <typename T>
int adam_multi_t(int nt, void *const *p, const void *const *g, void *const *m, void *const *v,
                 const int64_t *sizes, const AdamConsts<T> &k, const int32_t *decay, hipStream_t s,
                 ScheduleHeader *sched = nullptr)
{
    constexpr int VEC = VecOf<T>::N;
    constexpr int64_t kTile = (int64_t)kBlock * VEC * kUnroll;
    for (int i = 0; i < nt; i++)
        if (sizes[i] < 0 || (sizes[i] > 0 && (!p[i] || !g[i] || !m[i] || !v[i]))) return ZENU_ERR_ARG;
    for (int i = 0; i < nt; i++)
        if (adam_arrays_overlap(p[i], g[i], m[i], v[i], (size_t)sizes[i] * sizeof(T))) return ZENU_ERR_ARG;
    int i = 0;
    while (i < nt) {
        MultiArgs a;
        a.count = 0;
        int64_t blocks = 0;
        while (i < nt && a.count < kMaxMulti) {
            const int64_t tiles = (sizes[i] + kTile - 1) / kTile;
            if (tiles == 0) { i++; continue; }
            if (blocks + tiles > 0x7fffffffLL) {
                if (a.count == 0) return ZENU_ERR_UNSUPPORTED;
                break;
            }
            MultiEntry &e = a.e[a.count];
            e.p = p[i];
            e.g = g[i];
            e.m = m[i];
            e.v = v[i];
            e.n = sizes[i];
            e.decay = decay ? decay[i] : 0;
            e.vec_ok = aligned16(p[i]) && aligned16(g[i]) && aligned16(m[i]) && aligned16(v[i]);
            a.first_block[a.count] = (int32_t)blocks;
            blocks += tiles;
            a.count++;
            i++;
        }
        if (a.count == 0) break;
        a.first_block[a.count] = (int32_t)blocks;
        adam_multi_kernel<T, VEC><<<(unsigned)blocks, kBlock, 0, s>>>(a, k, sched);
        ZENU_LAUNCH_CHECK();
    }
    if (sched) {
        schedule_advance_kernel<<<1, 1, 0, s>>>(sched);
        ZENU_LAUNCH_CHECK();
    }
    return ZENU_OK;
}

template <typename T>
int sgd_multi_t(int nt, void *const *p, const void *const *g, const int64_t *sizes, T lr, hipStream_t s)
{
    constexpr int VEC = VecOf<T>::N;
    constexpr int64_t kTile = (int64_t)kBlock * VEC * kSgdUnroll;
    for (int i = 0; i < nt; i++)
        if (sizes[i] < 0 || (sizes[i] > 0 && (!p[i] || !g[i]))) return ZENU_ERR_ARG;
    for (int i = 0; i < nt; i++)
        if (ranges_overlap(p[i], (size_t)sizes[i] * sizeof(T), g[i], (size_t)sizes[i] * sizeof(T))) return ZENU_ERR_ARG;
    int i = 0;
    while (i < nt) {
        MultiArgs a;
        a.count = 0;
        int64_t blocks = 0;
        while (i < nt && a.count < kMaxMulti) {
            const int64_t tiles = (sizes[i] + kTile - 1) / kTile;
            if (tiles == 0) { i++; continue; }
            if (blocks + tiles > 0x7fffffffLL) {
                if (a.count == 0) return ZENU_ERR_UNSUPPORTED;
                break;
            }
            MultiEntry &e = a.e[a.count];
            e.p = p[i];
            e.g = g[i];
            e.m = nullptr;
            e.v = nullptr;
            e.n = sizes[i];
            e.decay = 0;
            e.vec_ok = aligned16(p[i]) && aligned16(g[i]);
            a.first_block[a.count] = (int32_t)blocks;
            blocks += tiles;
            a.count++;
            i++;
        }
        if (a.count == 0) break;
        a.first_block[a.count] = (int32_t)blocks;
        sgd_multi_kernel<T, VEC><<<(unsigned)blocks, kBlock, 0, s>>>(a, lr);
        ZENU_LAUNCH_CHECK();
    }
    return ZENU_OK;
}

}  // namespace
}  // namespace zenu

using namespace zenu;

extern "C" {

int zenu_hip_sgd_step_multi(int dtype, int n_tensors, void *const *p_dev, const void *const *g_dev,
                            const int64_t *sizes, double lr, zenu_stream_t stream)
{
    if (n_tensors < 0) return ZENU_ERR_ARG;
    if (n_tensors == 0) return ZENU_OK;
    if (!p_dev || !g_dev || !sizes) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    if (dtype == ZENU_F32) return sgd_multi_t<float>(n_tensors, p_dev, g_dev, sizes, (float)lr, as_stream(stream));
    if (dtype == ZENU_F64) return sgd_multi_t<double>(n_tensors, p_dev, g_dev, sizes, lr, as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_sgd_step(int dtype, void *p_dev, const void *g_dev, int64_t n, double lr, zenu_stream_t stream)
{
    if (n < 0 || (n > 0 && (!p_dev || !g_dev))) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    if (n == 0) return ZENU_OK;
    if (ranges_overlap(p_dev, (size_t)n * (dtype == ZENU_F64 ? 8 : 4), g_dev, (size_t)n * (dtype == ZENU_F64 ? 8 : 4)))
        return ZENU_ERR_ARG;
    hipStream_t s = as_stream(stream);
    const bool vec = aligned16(p_dev) && aligned16(g_dev);
    if (dtype == ZENU_F32) {
        const int v = vec ? 4 : 1;
        const int64_t tile = (int64_t)kBlock * v * 4;
        const int64_t grid = (n + tile - 1) / tile;
        if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
        if (vec) sgd_kernel<float, 4><<<(unsigned)grid, kBlock, 0, s>>>((float *)p_dev, (const float *)g_dev, n, (float)lr);
        else     sgd_kernel<float, 1><<<(unsigned)grid, kBlock, 0, s>>>((float *)p_dev, (const float *)g_dev, n, (float)lr);
    } else if (dtype == ZENU_F64) {
        const int v = vec ? 2 : 1;
        const int64_t tile = (int64_t)kBlock * v * 4;
        const int64_t grid = (n + tile - 1) / tile;
        if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
        if (vec) sgd_kernel<double, 2><<<(unsigned)grid, kBlock, 0, s>>>((double *)p_dev, (const double *)g_dev, n, lr);
        else     sgd_kernel<double, 1><<<(unsigned)grid, kBlock, 0, s>>>((double *)p_dev, (const double *)g_dev, n, lr);
    } else {
        return ZENU_ERR_ARG;
    }
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

int zenu_hip_adamw_step(int dtype, void *p_dev, const void *g_dev, void *m_dev, void *v_dev, int64_t n,
                        double lr, double beta1, double beta2, double eps, double weight_decay,
                        int apply_decay, double step, zenu_stream_t stream)
{
    if (n < 0 || (n > 0 && (!p_dev || !g_dev || !m_dev || !v_dev))) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    if (dtype == ZENU_F32)
        return adam_t<float>(p_dev, g_dev, m_dev, v_dev, n,
                             make_consts<float>(lr, beta1, beta2, eps, weight_decay, step), apply_decay,
                             as_stream(stream));
    if (dtype == ZENU_F64)
        return adam_t<double>(p_dev, g_dev, m_dev, v_dev, n,
                              make_consts<double>(lr, beta1, beta2, eps, weight_decay, step), apply_decay,
                              as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_adam_step(int dtype, void *p_dev, const void *g_dev, void *m_dev, void *v_dev, int64_t n,
                       double lr, double beta1, double beta2, double eps, double step, zenu_stream_t stream)
{
    return zenu_hip_adamw_step(dtype, p_dev, g_dev, m_dev, v_dev, n, lr, beta1, beta2, eps, 0.0, 0, step,
                               stream);
}

int zenu_hip_adam_step_multi(int dtype, int n_tensors, void *const *p_dev, const void *const *g_dev,
                             void *const *m_dev, void *const *v_dev, const int64_t *sizes, double lr,
                             double beta1, double beta2, double eps, double weight_decay,
                             const int32_t *apply_decay, double step, zenu_stream_t stream)
{
    if (n_tensors < 0) return ZENU_ERR_ARG;
    if (n_tensors == 0) return ZENU_OK;
    if (!p_dev || !g_dev || !m_dev || !v_dev || !sizes) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    if (dtype == ZENU_F32)
        return adam_multi_t<float>(n_tensors, p_dev, g_dev, m_dev, v_dev, sizes,
                                   make_consts<float>(lr, beta1, beta2, eps, weight_decay, step),
                                   apply_decay, as_stream(stream));
    if (dtype == ZENU_F64)
        return adam_multi_t<double>(n_tensors, p_dev, g_dev, m_dev, v_dev, sizes,
                                    make_consts<double>(lr, beta1, beta2, eps, weight_decay, step),
                                    apply_decay, as_stream(stream));
    return ZENU_ERR_ARG;
}

// host side of a schedule (the handle the C ABI passes around)
struct AdamScheduleHost {
    ScheduleHeader *dev;
    int dtype;
    double beta1, beta2;
    int64_t first_step;
    int n_steps;
};

int zenu_hip_adam_schedule_create(void **schedule, int dtype, double beta1, double beta2, int64_t first_step,
                                  int n_steps, zenu_stream_t stream)
{
    if (!schedule || first_step < 1 || n_steps < 1 || n_steps > (1 << 24)) return ZENU_ERR_ARG;
    if (dtype != ZENU_F32 && dtype != ZENU_F64) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    hipStream_t s = as_stream(stream);
    hipStreamCaptureStatus cs = hipStreamCaptureStatusNone;
    if (s && hipStreamIsCapturing(s, &cs) == hipSuccess && cs != hipStreamCaptureStatusNone) return ZENU_ERR_UNSUPPORTED;
    const size_t esz = dtype == ZENU_F32 ? 4 : 8;
    const size_t bytes = sizeof(ScheduleHeader) + (size_t)n_steps * 2 * esz;
    std::vector<unsigned char> host(bytes);
    ScheduleHeader *h = reinterpret_cast<ScheduleHeader *>(host.data());
    h->cursor = 0;
    h->n = (uint32_t)n_steps;
    h->exhausted = 0;
    h->pad = 0;
    for (int i = 0; i < n_steps; i++) {
        const double step = (double)(first_step + i);
        if (dtype == ZENU_F32) {
            const AdamConsts<float> k = make_consts<float>(0, beta1, beta2, 0, 0, step);
            float *t = reinterpret_cast<float *>(h + 1);
            t[2 * i] = k.c1;
            t[2 * i + 1] = k.c2;
        } else {
            const AdamConsts<double> k = make_consts<double>(0, beta1, beta2, 0, 0, step);
            double *t = reinterpret_cast<double *>(h + 1);
            t[2 * i] = k.c1;
            t[2 * i + 1] = k.c2;
        }
    }
    void *dev = nullptr;
    rc = zenu_hip_raw_malloc(&dev, bytes);
    if (rc) return rc;
    rc = zenu_hip_memcpy_h2d(dev, host.data(), bytes, stream);   // blocking: `host` may go
    if (rc) {
        (void)zenu_hip_raw_free(dev);
        return rc;
    }
    AdamScheduleHost *hs = new AdamScheduleHost;
    hs->dev = static_cast<ScheduleHeader *>(dev);
    hs->dtype = dtype;
    hs->beta1 = beta1;
    hs->beta2 = beta2;
    hs->first_step = first_step;
    hs->n_steps = n_steps;
    *schedule = hs;
    return ZENU_OK;
}

int zenu_hip_adam_schedule_destroy(void *schedule, zenu_stream_t stream)
{
    if (!schedule) return ZENU_OK;
    AdamScheduleHost *hs = static_cast<AdamScheduleHost *>(schedule);
    ZENU_HIP_TRY(hipStreamSynchronize(as_stream(stream)));   // the updates that read it are done
    int rc = zenu_hip_raw_free(hs->dev);
    delete hs;
    return rc;
}

int zenu_hip_adam_schedule_query(void *schedule, int64_t *next_step, int64_t *steps_left, int64_t *refused,
                                 zenu_stream_t stream)
{
    if (!schedule) return ZENU_ERR_ARG;
    AdamScheduleHost *hs = static_cast<AdamScheduleHost *>(schedule);
    ScheduleHeader h;
    int rc = zenu_hip_memcpy_d2h(&h, hs->dev, sizeof h, stream);   // blocking
    if (rc) return rc;
    if (next_step) *next_step = hs->first_step + h.cursor;
    if (steps_left) *steps_left = (int64_t)h.n - h.cursor;
    if (refused) *refused = h.exhausted;
    return ZENU_OK;
}

int zenu_hip_adam_step_multi_scheduled(int dtype, int n_tensors, void *const *p_dev, const void *const *g_dev,
                                       void *const *m_dev, void *const *v_dev, const int64_t *sizes, double lr,
                                       double eps, double weight_decay, const int32_t *apply_decay,
                                       void *schedule, zenu_stream_t stream)
{
    if (n_tensors < 0 || !schedule) return ZENU_ERR_ARG;
    AdamScheduleHost *hs = static_cast<AdamScheduleHost *>(schedule);
    if (hs->dtype != dtype) return ZENU_ERR_ARG;
    if (n_tensors > 0 && (!p_dev || !g_dev || !m_dev || !v_dev || !sizes)) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    // the step-dependent scalars come from the table; everything else as in the eager call
    if (dtype == ZENU_F32)
        return adam_multi_t<float>(n_tensors, p_dev, g_dev, m_dev, v_dev, sizes,
                                   make_consts<float>(lr, hs->beta1, hs->beta2, eps, weight_decay, 1.0),
                                   apply_decay, as_stream(stream), hs->dev);
    return adam_multi_t<double>(n_tensors, p_dev, g_dev, m_dev, v_dev, sizes,
                                make_consts<double>(lr, hs->beta1, hs->beta2, eps, weight_decay, 1.0),
                                apply_decay, as_stream(stream), hs->dev);
}

}  // extern "C"
