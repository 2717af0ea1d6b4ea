// reduce.hip -- axis reductions for gfx950: sum, asum, max, arg-max (first index wins ties).
//
// The reference reduces by host recursion: `sum` issues shape[axis] whole-slice `+=` launches
// (zenu-matrix/src/operation/sum.rs:12-31) and `max_axis` one alloc + copy + kernel + two
// blocking single-element copies per output element (zenu-matrix/src/operation/max.rs:45-99).
// Here the source is addressed as [outer, R, inner] with R the reduced axis (any view whose kept
// dims form one uniform stride chain plus a unit-stride run; other views are copied first) and
// one of two kernels runs:
//
//   rows : inner < 16, normally 1 (the reduced axis is contiguous) -- one workgroup (or one
//          wavefront when the row is short) per row, 128-bit loads, four independent
//          accumulators per lane (eight when workgroups share a row), wave64 butterfly built
//          from DPP (quad_perm, row_half_mirror, row_mirror), ds_swizzle and one cross-half
//          exchange, then a fixed-order combine of the 4 waves through LDS.
//   cols : inner >= 16 -- a 32 x 8 thread tile: 32 lanes own 32 column vectors (512-byte row
//          pieces, coalesced 128-bit loads), 8 row lanes walk the reduced axis with four rows in
//          flight each, combined through LDS in fixed order.
//
// Both kernels can split the reduced axis over several workgroups; the splits interleave chunk
// by chunk so the grid sweeps the source as one window.  Partial results go to a small
// workspace; each workgroup then bumps an arrival counter (a two-level tree of counters when
// many workgroups share an output) and the one that arrives last folds the partials of its
// outputs, always in split order.  No workgroup waits for another and no atomic touches data:
// the combination tree is fixed by the launch geometry, so results are bit-reproducible, and
// the whole reduction is ONE launch.
//
// Arg-max follows MaxIdx for Cpu (max.rs:19-34): start from element 0 and replace on strict '>'.
// That is "largest value, lowest index on ties", except for NaN: a NaN at position 0 is never
// replaced, a NaN anywhere else never replaces.  Mapping NaN to +inf at position 0 and to -inf
// elsewhere turns the scan into an associative, commutative (key, index) maximum that any tree
// reproduces; the value written is re-read from the source at the winning index so its bits
// (NaN payload, sign of zero) are the source's.
#include <math.h>

#include <type_traits>

#include "common.hpp"
#include "vecmem.hpp"

namespace zenu {

// `n` consecutive arrival counters (zero at rest) from the ring of `stream`, or nullptr
int *reserve_counters(int64_t n, hipStream_t stream);
// `nwords` tagged 64-bit words from the ring of `stream` and this launch's tag, or nullptr
uint64_t *reserve_slots(int64_t nwords, hipStream_t stream, uint32_t *epoch);
int reduce_spin_limit();
bool rehearsal_needed(size_t bytes, hipStream_t stream);
bool library_ready();

namespace {

// ---- static scratch of the allocation-free entry point (zenu_hip_sum_axis_noalloc) -------------------
// Counters, partials and the staging of a strided destination for callers that may not allocate.
// Held by the device from the moment the library's code object is loaded until the process ends.
// In host code the array's name is only a stand-in: its device address comes from
// hipGetSymbolAddress (init_static_scratch, called once by the library's init with the device
// current) and that pointer is what kernels and fills get.
constexpr size_t kScratchCounters = 4096;                       // arrival counters (ints)
constexpr size_t kScratchCounterBytes = kScratchCounters * sizeof(int);
constexpr size_t kScratchPartialBytes = 512u << 10;             // partial results of a split reduction
constexpr size_t kScratchStageBytes = 512u << 10;               // contiguous result of a strided destination
constexpr size_t kScratchBytes = kScratchCounterBytes + kScratchPartialBytes + kScratchStageBytes;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
unsigned char *g_scratch_ptr = nullptr;   // device address of `scratch` (one device per process)

// How often a folding workgroup gave up polling and computed missing partials itself (see "hand-off
// through tagged words").  Such a launch is correct but slow, and nothing else would show it.
static __device__ unsigned int fold_fallbacks;
unsigned int *g_fold_fallbacks_ptr = nullptr;   // device address of `fold_fallbacks`

// where a reduction finds its cross-workgroup memory when it may not allocate
struct FixedScratch {
    int *counters;
    int64_t n_counters;
    void *partials;
    size_t partial_bytes;
    void *stage;
    size_t stage_bytes;
};

constexpr int kBlock = 256;
constexpr int kWave = 64;
constexpr int kWaves = kBlock / kWave;
#ifndef ZENU_SPLIT_U
#define ZENU_SPLIT_U 8
#endif
constexpr int kSlotBatch = 2;           // partial results a thread of the folding workgroup polls for at a time
constexpr int kRowsU = 4;               // vectors in flight per lane, one workgroup or wavefront per row
constexpr int kSplitU = ZENU_SPLIT_U;   // the same when workgroups share a row


// ---- wave64 exchange primitives (word-wise so any POD accumulator works) ---------------------------

template <int CTRL> __device__ __forceinline__ int dpp_word(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}

enum { kDppXor1 = 0xB1, kDppXor2 = 0x4E, kDppHalfMirror = 0x141, kDppMirror = 0x140 };

template <typename A, typename WordFn> __device__ __forceinline__ A map_words(A v, WordFn fn)
{
    static_assert(sizeof(A) % 4 == 0, "accumulator must be a multiple of 4 bytes");
    constexpr int W = sizeof(A) / 4;
    int w[W];
    __builtin_memcpy(w, &v, sizeof(A));
#pragma unroll
    for (int i = 0; i < W; i++) w[i] = fn(w[i]);
    A r;
    __builtin_memcpy(&r, w, sizeof(A));
    return r;
}

// After this every lane of the wavefront holds the reduction of all 64 lanes.  The merge
// operator must be commutative so both partners compute identical bits.
template <typename Tr> __device__ __forceinline__ typename Tr::Acc wave_allreduce(typename Tr::Acc a)
{
    typedef typename Tr::Acc A;
    a = Tr::merge(a, map_words<A>(a, [](int w) { return dpp_word<kDppXor1>(w); }));
    a = Tr::merge(a, map_words<A>(a, [](int w) { return dpp_word<kDppXor2>(w); }));
    a = Tr::merge(a, map_words<A>(a, [](int w) { return dpp_word<kDppHalfMirror>(w); }));
    a = Tr::merge(a, map_words<A>(a, [](int w) { return dpp_word<kDppMirror>(w); }));
    // lane ^ 16 inside each half: ds_swizzle bit mode (and 0x1f, or 0, xor 0x10)
    a = Tr::merge(a, map_words<A>(a, [](int w) { return __builtin_amdgcn_ds_swizzle(w, 0x401F); }));
    // lane ^ 32: the two halves of the wavefront
    a = Tr::merge(a, map_words<A>(a, [](int w) { return __shfl_xor(w, 32, kWave); }));
    return a;
}

// Block-wide reduction; the result is valid in every thread.
template <typename Tr> __device__ __forceinline__ typename Tr::Acc block_allreduce(typename Tr::Acc a)
{
    typedef typename Tr::Acc A;
    __shared__ A lds[kWaves];
    a = wave_allreduce<Tr>(a);
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x & (kWave - 1)) == 0) lds[wave] = a;
    __syncthreads();
    A r = lds[0];
#pragma unroll
    for (int w = 1; w < kWaves; w++) r = Tr::merge(r, lds[w]);
    __syncthreads();
    return r;
}

// ---- accumulator traits ------------------------------------------------------------------------------

// Accumulator traits.  `update` folds the next element (in increasing position order) into a
// lane's accumulator and is the only code in the per-element hot loop; `merge` combines two
// accumulators (lanes, waves, workgroups) and must be commutative and associative.
template <typename T> struct SumTr {
    typedef T Acc;
    static constexpr bool kHasIdx = false;
    __device__ __forceinline__ static Acc identity() { return (T)0; }
    __device__ __forceinline__ static Acc update(Acc a, T x, int64_t) { return a + x; }
    __device__ __forceinline__ static Acc first(Acc a, T) { return a; }
    __device__ __forceinline__ static Acc from_partial(T x, int64_t) { return x; }
    __device__ __forceinline__ static Acc merge(Acc a, Acc b) { return a + b; }
    __device__ __forceinline__ static T key(Acc a) { return a; }
    __device__ __forceinline__ static int64_t idx(Acc) { return 0; }
};

template <typename T> struct AsumTr : SumTr<T> {
    __device__ __forceinline__ static T update(T a, T x, int64_t) { return a + fabs(x); }
};

template <typename T> struct ArgPair {
    T key;
    int32_t idx;
};

// Arg-max with the semantics of the sequential scan of max.rs:23-31.
//   * In a lane, elements arrive in increasing position, so "replace on strict >" keeps the first
//     index, ignores NaN (NaN > key is false) and costs one compare and two selects.
//   * -inf elements never pass the strict test against the -inf identity; if nothing does, every
//     element is -inf or NaN and the scan would have stayed at index 0: idx() maps the untouched
//     identity index to 0.
//   * A NaN at position 0 is never replaced by the scan: first() turns it into a +inf key at
//     index 0, which no later element beats and which wins every tie by index.
constexpr int32_t kNoIdx = 0x7fffffff;
template <typename T> struct ArgmaxTr {
    typedef ArgPair<T> Acc;
    static constexpr bool kHasIdx = true;
    __device__ __forceinline__ static Acc identity()
    {
        Acc a;
        a.key = -INFINITY;
        a.idx = kNoIdx;
        return a;
    }
    __device__ __forceinline__ static Acc update(Acc a, T x, int64_t pos)
    {
        const bool gt = x > a.key;
        a.key = gt ? x : a.key;
        a.idx = gt ? (int32_t)pos : a.idx;
        return a;
    }
    // `x` is the element at position 0 of the reduced axis, already folded in by update()
    __device__ __forceinline__ static Acc first(Acc a, T x)
    {
        if (x != x) {
            a.key = INFINITY;
            a.idx = 0;
        }
        return a;
    }
    __device__ __forceinline__ static Acc from_partial(T k, int64_t i)
    {
        Acc a;
        a.key = k;
        a.idx = (int32_t)i;
        return a;
    }
    __device__ __forceinline__ static Acc merge(Acc a, Acc b)
    {
        const bool take_b = (b.key > a.key) || (b.key == a.key && b.idx < a.idx);
        return take_b ? b : a;
    }
    __device__ __forceinline__ static T key(Acc a) { return a.key; }
    __device__ __forceinline__ static int64_t idx(Acc a) { return a.idx == kNoIdx ? 0 : a.idx; }
};

// ---- kernel parameters ---------------------------------------------------------------------------------

template <typename T> struct RedParams {
    const T *in;
    // geometry: output element o = (q, c) with q = o / inner, c = o % inner;
    // its R values sit at in[q * outer_stride + c + r * elem_stride]
    int64_t nout;            // number of outputs = outer * inner
    int64_t R;               // reduced length
    int64_t inner;
    int64_t outer_stride;
    int64_t elem_stride;
    int splits;              // workgroups along R
    int cols_shift;          // column kernels: log2 of the lanes along the columns (chosen by the host)
    // results
    T *out_val;              // final value (may be null)
    int64_t *out_idx;        // final index (may be null)
    // cross-workgroup stage (splits > 1): partial results and one arrival counter per group of
    // workgroups that share outputs; the counters are zero at rest
    T *part_key;
    int32_t *part_idx;
    int *counters;
    int fan;                 // splits per leaf counter of the arrival tree
    int cstride;             // counters per group: 1 + number of leaves (1 when fan >= splits)
    // the other cross-workgroup stage: tagged words (slots != null), see "hand-off through tagged words"
    uint64_t *slots;
    uint32_t epoch;          // this launch's tag, never zero
    int spin_limit;          // polls before the folding workgroup computes what is missing itself
    unsigned int *fallbacks; // bumped once per batch of partials that the folding workgroup had to compute
    // optional transform of the source on its way in (column kernels, vector path, sums only):
    // the reduced value is in[i] * (pre_x[i] > 0 ? 1 : pre_alpha * -1), the gradient of ReLU
    // (zenu-autograd/src/activation/relu.rs:35-44), which is also stored to pre_out[i]; the three
    // arrays share the source's layout.  Every source element is loaded by exactly one thread of
    // the launch, so every element of pre_out is written once.
    const T *pre_x;
    T *pre_out;
    T pre_alpha;
    // value gather for max: value = gsrc[q * g_outer_stride + c + idx * g_elem_stride]
    const T *gsrc;
    int64_t g_outer_stride, g_elem_stride;
};

template <typename T, typename Tr>
__device__ __forceinline__ void emit_final(const RedParams<T> &p, int64_t o, typename Tr::Acc r)
{
    if (Tr::kHasIdx) {
        if (p.out_idx) p.out_idx[o] = Tr::idx(r);
        if (p.out_val) {
            const int64_t q = o / p.inner, c = o - q * p.inner;
            p.out_val[o] = p.gsrc[q * p.g_outer_stride + c + Tr::idx(r) * p.g_elem_stride];
        }
    } else {
        p.out_val[o] = Tr::key(r);
    }
}

// Cross-workgroup hand-off.  The workgroups of one launch run on 8 XCDs with separate L2s, so the
// partials travel with device-scope (write-through / L2-bypassing) accesses instead of a
// device-scope fence: a release fence would write back and invalidate the whole L2 in every
// workgroup (measured: 20x slower).  Order of events in a producer: device-scope stores of the
// partials (write-through: they go to memory, not to this XCD's L2); every thread then waits
// until its own vector-memory operations are acknowledged (an explicit s_waitcnt vmcnt(0): a
// workgroup-scope release fence only waits for LDS and scalar traffic and would let the counter
// overtake the partials); barrier; one device-scope atomic increment by thread 0.  A store that
// has been acknowledged at device scope has reached the point every XCD reads through, so the
// consumer (the workgroup that reads expected-1 from the counter) sees it with device-scope
// loads, which it issues only after that atomic has returned.
template <typename U> __device__ __forceinline__ void store_agent(U *p, U v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <typename U> __device__ __forceinline__ U load_agent(const U *p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T, typename Tr>
__device__ __forceinline__ void emit_partial(const RedParams<T> &p, int64_t slot, typename Tr::Acc r)
{
    const T k = Tr::key(r);
    if constexpr (sizeof(T) == 4) {
        uint32_t u;
        __builtin_memcpy(&u, &k, 4);
        store_agent(reinterpret_cast<uint32_t *>(p.part_key + slot), u);
    } else {
        uint64_t u;
        __builtin_memcpy(&u, &k, 8);
        store_agent(reinterpret_cast<uint64_t *>(p.part_key + slot), u);
    }
    if (Tr::kHasIdx) store_agent(p.part_idx + slot, (int32_t)Tr::idx(r));  // only -inf/NaN: (-inf, 0)
}

template <typename T, typename Tr>
__device__ __forceinline__ typename Tr::Acc load_partial(const RedParams<T> &p, int64_t slot)
{
    T k;
    if constexpr (sizeof(T) == 4) {
        uint32_t u = load_agent(reinterpret_cast<const uint32_t *>(p.part_key + slot));
        __builtin_memcpy(&k, &u, 4);
    } else {
        uint64_t u = load_agent(reinterpret_cast<const uint64_t *>(p.part_key + slot));
        __builtin_memcpy(&k, &u, 8);
    }
    int32_t i = 0;
    if (Tr::kHasIdx) i = load_agent(p.part_idx + slot);
    return Tr::from_partial(k, i);
}

// a vector of the source; with PRE the ReLU-gradient transform described at RedParams::pre_x
template <typename T, int VEC, bool NT, bool PRE>
__device__ __forceinline__ Pack<T, VEC> load_src(const RedParams<T> &p, const T *ptr)
{
    Pack<T, VEC> g = load_pack<T, VEC, NT>(ptr);
    if constexpr (PRE) {
        const int64_t off = ptr - p.in;
        const Pack<T, VEC> x = load_pack<T, VEC, NT>(p.pre_x + off);
#pragma unroll
        for (int j = 0; j < VEC; j++) g.v[j] = g.v[j] * ((x.v[j] > (T)0) ? (T)1 : p.pre_alpha * (T)-1);
        store_pack<T, VEC, NT>(p.pre_out + off, g);
    }
    return g;
}

// ---- hand-off through tagged words ---------------------------------------------------------------------
// The faster of the two cross-workgroup stages (whole-tensor f32 sum of 128 MiB: 21.5 us against
// 23.4 us with the counters; streaming alone takes 20.4 us).  The counters cost four dependent
// device-scope round trips after the last workgroup has finished streaming (partial stored and
// acknowledged, leaf counter, root counter, partials loaded).  Here a partial travels as 64-bit
// words {tag, 32 bits of payload}, each stored with ONE device-scope store and valid by itself: the
// tag is this launch's number on its stream (RedParams::epoch), which no word left in the ring by
// an earlier launch carries.  The workgroup with the highest index of a group -- workgroups are
// dispatched in index order, so the others are running or done when it starts -- folds: after its
// own streaming it polls the group's words until every tag matches and merges in split order.
// What is left on the critical path is one store in flight and one poll.
// Nothing here depends on the dispatch order for correctness: after `spin_limit` fruitless polls
// the folding workgroup computes the missing partials itself, exactly as their owners would, and
// stores them; a late owner later stores the same bits again.  Nobody else ever waits.
// Launches recorded into a graph would replay their tag, so they use the counters; so do requests
// larger than half a stream's ring of words, the allocation-free entry point, and the column
// kernel (see reduce_strided).

template <typename T, typename Tr> struct SlotWords {
    static constexpr int K = sizeof(T) / 4;                    // payload words of the key
    static constexpr int W = K + (Tr::kHasIdx ? 1 : 0);        // plus the index
};

// word w of slot s lives at slots[w * nslots + s]: consecutive slots are consecutive words
template <typename T, typename Tr>
__device__ __forceinline__ void emit_slot(const RedParams<T> &p, int64_t nslots, int64_t s, typename Tr::Acc r)
{
    const T k = Tr::key(r);
    uint32_t w[3];
    __builtin_memcpy(w, &k, sizeof(T));
    if (Tr::kHasIdx) w[SlotWords<T, Tr>::K] = (uint32_t)Tr::idx(r);
    const uint64_t tag = (uint64_t)p.epoch << 32;
#pragma unroll
    for (int i = 0; i < SlotWords<T, Tr>::W; i++) store_agent(p.slots + i * nslots + s, tag | w[i]);
}

// false while any word of the slot still carries another tag
template <typename T, typename Tr>
__device__ __forceinline__ bool load_slot(const RedParams<T> &p, int64_t nslots, int64_t s, typename Tr::Acc &r)
{
    uint32_t w[3];
    bool ok = true;
#pragma unroll
    for (int i = 0; i < SlotWords<T, Tr>::W; i++) {
        const uint64_t v = load_agent(p.slots + i * nslots + s);
        ok = ok && (uint32_t)(v >> 32) == p.epoch;
        w[i] = (uint32_t)v;
    }
    T k;
    __builtin_memcpy(&k, w, sizeof(T));
    r = Tr::from_partial(k, Tr::kHasIdx ? (int32_t)w[SlotWords<T, Tr>::K] : 0);
    return ok;
}

// Called by every thread of a workgroup after its partials are stored.  Returns true in the one
// workgroup of the group that arrives last; it performs the fold.  No workgroup waits for
// another.  Atomics of many workgroups on ONE address are served one after the other (measured:
// about 12 ns each, 6 us for 512 workgroups that finish together), so arrival is a two-level
// tree: `fan` consecutive splits share a leaf counter and the last one at a leaf moves on to the
// root.  `c` points at the group's 1 + ceil(splits / fan) counters (root first); with
// fan >= splits only the root is used.  Leaves are reset by their last arriver, the root by
// the folding workgroup.
__device__ __forceinline__ bool arrive_last(int *c, int split, int splits, int fan)
{
    __shared__ int s_last;
    // every thread: all of my vector-memory stores (the partials) are acknowledged before the
    // barrier lets thread 0 announce this workgroup
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        bool last;
        if (fan >= splits) {
            last = __hip_atomic_fetch_add(c, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == splits - 1;
        } else {
            const int leaves = (splits + fan - 1) / fan;
            const int leaf = split / fan;
            const int members = (leaf == leaves - 1) ? splits - leaf * fan : fan;
            last = false;
            if (__hip_atomic_fetch_add(c + 1 + leaf, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == members - 1) {
                store_agent(c + 1 + leaf, 0);
                last = __hip_atomic_fetch_add(c, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == leaves - 1;
            }
        }
        s_last = last;
    }
    __syncthreads();
    return s_last != 0;
}

// ---- kernel A: rows --------------------------------------------------------------------------------------
// VEC > 1 requires elem_stride == 1, 16-byte aligned rows (checked on the host).
// WAVE_ROW: one wavefront per output (4 outputs per workgroup, never split), otherwise one
// workgroup per (output, split); with splits > 1 the last workgroup of an output to finish folds
// that output's partials in a fixed order.

enum { kWaveRow = 0, kBlockRow = 1, kSplitRow = 2 };

template <typename T, typename Tr, int VEC, int MODE, bool NT, int U>
__global__ __launch_bounds__(kBlock) void reduce_rows_kernel(RedParams<T> p)
{
    typedef typename Tr::Acc A;
    constexpr bool WAVE_ROW = MODE == kWaveRow;
    const int nsplit = MODE == kSplitRow ? p.splits : 1;
    const int lane_n = WAVE_ROW ? kWave : kBlock;
    const int lane = WAVE_ROW ? (threadIdx.x & (kWave - 1)) : threadIdx.x;
    int64_t o;
    int my_split;
    if (WAVE_ROW) {
        o = (int64_t)blockIdx.x * kWaves + threadIdx.x / kWave;
        my_split = 0;
    } else if (MODE == kBlockRow) {
        o = blockIdx.x;
        my_split = 0;
    } else {            // grid = (splits, outputs): no division at the start of a workgroup
        o = blockIdx.y;
        my_split = (int)blockIdx.x;
    }
    const bool active = o < p.nout;

    // what this lane accumulates of split `split` of output o, the U accumulators merged in a fixed tree
    auto lane_partial = [&](int split) -> A {
        A acc[U];
#pragma unroll
        for (int u = 0; u < U; u++) acc[u] = Tr::identity();
        if (active) {
            int64_t q = o, c = 0;
            if (p.inner != 1) {
                q = o / p.inner;
                c = o - q * p.inner;
            }
            const int64_t base = q * p.outer_stride + c;
            // The splits of an output interleave chunk by chunk (split s takes chunks s, s + splits,
            // ...), so the workgroups of a launch sweep the source together as one moving window
            // instead of each streaming its own far-apart segment in lockstep.
            const int64_t R = p.R;
            if (VEC > 1) {
                const T *row = p.in + base;
                const int64_t step = (int64_t)lane_n * VEC;
                const int64_t chunk = U * step;
                const int64_t stride = chunk * nsplit;
                for (int64_t b = (int64_t)split * chunk; b < R; b += stride) {
                    int64_t r = b + (int64_t)lane * VEC;
                    if (b + chunk <= R) {      // U vectors in flight per lane
                        Pack<T, VEC> x[U];
#pragma unroll
                        for (int u = 0; u < U; u++) x[u] = load_pack<T, VEC, NT>(row + r + u * step);
#pragma unroll
                        for (int u = 0; u < U; u++) {
#pragma unroll
                            for (int j = 0; j < VEC; j++) acc[u] = Tr::update(acc[u], x[u].v[j], r + u * step + j);
                        }
                    } else {                   // the last, partial chunk of the row
                        for (; r + VEC <= R; r += step) {
                            Pack<T, VEC> x = load_pack<T, VEC, false>(row + r);
#pragma unroll
                            for (int j = 0; j < VEC; j++) acc[0] = Tr::update(acc[0], x.v[j], r + j);
                        }
                        if (r < R)             // ragged end (R % VEC != 0): one lane
                            for (int j = 0; r + j < R; j++) acc[0] = Tr::update(acc[0], row[r + j], r + j);
                    }
                }
                if (split == 0 && lane == 0) acc[0] = Tr::first(acc[0], row[0]);
            } else {
                const int64_t chunk = (int64_t)U * lane_n;
                const int64_t stride = chunk * nsplit;
                for (int64_t b = (int64_t)split * chunk; b < R; b += stride) {
                    int64_t r = b + lane;
                    if (b + chunk <= R) {
#pragma unroll
                        for (int u = 0; u < U; u++) {
                            const int64_t rr = r + (int64_t)u * lane_n;
                            acc[u] = Tr::update(acc[u], p.in[base + rr * p.elem_stride], rr);
                        }
                    } else {
                        for (; r < R; r += lane_n) acc[0] = Tr::update(acc[0], p.in[base + r * p.elem_stride], r);
                    }
                }
                if (split == 0 && lane == 0) acc[0] = Tr::first(acc[0], p.in[base]);
            }
        }
        // fixed tree over the U accumulators
#pragma unroll
        for (int w = 1; w < U; w *= 2) {
#pragma unroll
            for (int u = 0; u + w < U; u += 2 * w) acc[u] = Tr::merge(acc[u], acc[u + w]);
        }
        return acc[0];
    };

    A a = lane_partial(my_split);
    if (WAVE_ROW) {
        a = wave_allreduce<Tr>(a);
        if (active && lane == 0) emit_final<T, Tr>(p, o, a);
        return;
    }
    a = block_allreduce<Tr>(a);
    if (MODE != kSplitRow) {
        if (lane == 0) emit_final<T, Tr>(p, o, a);
        return;
    }
    const int splits = p.splits;
    A f = Tr::identity();
    if (p.slots) {
        // tagged words: store and leave; the workgroup with the highest index of the output folds
        const int64_t nslots = p.nout * splits;
        const int64_t s_base = o * splits;
        if (lane == 0) emit_slot<T, Tr>(p, nslots, s_base + my_split, a);
        if (my_split != splits - 1) return;
        // lane l takes splits l, l + 256, ... in batches of kSlotBatch (few registers: every workgroup
        // of the launch pays for what the folding one needs); merge in split order
        for (int s0 = 0; s0 < splits; s0 += kSlotBatch * kBlock) {
            A t[kSlotBatch];
            int polls = 0;
            bool force = p.spin_limit == 0;   // the host asks for the fallback itself: every partial of the batch
            for (;;) {
                int ok = 1;
#pragma unroll
                for (int u = 0; u < kSlotBatch; u++) {
                    const int sidx = s0 + lane + u * kBlock;
                    t[u] = Tr::identity();
                    if (sidx < splits && !load_slot<T, Tr>(p, nslots, s_base + sidx, t[u])) ok = 0;
                }
                if (__syncthreads_and(ok) && !force) break;
                if (force || ++polls > p.spin_limit) {
                    // compute what is still missing in this batch, as its owner would
                    if (lane == 0 && p.fallbacks)
                        __hip_atomic_fetch_add(p.fallbacks, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    const int s_end = s0 + kSlotBatch * kBlock < splits ? s0 + kSlotBatch * kBlock : splits;
                    for (int sp = s0; sp < s_end; sp++) {
                        A probe;
                        const int have = (!force && lane == 0 && load_slot<T, Tr>(p, nslots, s_base + sp, probe)) ? 1 : 0;
                        if (__syncthreads_or(have)) continue;
                        const A r = block_allreduce<Tr>(lane_partial(sp));
                        if (lane == 0) emit_slot<T, Tr>(p, nslots, s_base + sp, r);
                    }
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // the words are in place before the next poll
                    __syncthreads();
                    polls = 0;
                    force = false;
                }
            }
#pragma unroll
            for (int u = 0; u < kSlotBatch; u++) f = Tr::merge(f, t[u]);
        }
        f = block_allreduce<Tr>(f);
        if (lane == 0) emit_final<T, Tr>(p, o, f);
        return;
    }
    if (lane == 0) emit_partial<T, Tr>(p, o * splits + my_split, a);
    if (!arrive_last(p.counters + o * p.cstride, my_split, splits, p.fan)) return;
    // fold the splits of output o: lane l takes splits l, l + 256, ...; then the fixed block tree
    for (int s0 = lane; s0 < splits; s0 += 4 * kBlock) {
        A t[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {   // issue the loads together, merge in split order
            const int sidx = s0 + u * kBlock;
            t[u] = sidx < splits ? load_partial<T, Tr>(p, o * splits + sidx) : Tr::identity();
        }
#pragma unroll
        for (int u = 0; u < 4; u++) f = Tr::merge(f, t[u]);
    }
    f = block_allreduce<Tr>(f);
    if (lane == 0) {
        emit_final<T, Tr>(p, o, f);
        store_agent(p.counters + o * p.cstride, 0);   // back to rest for the next launch
    }
}

// ---- kernel B: cols ---------------------------------------------------------------------------------------
// Source [outer, R, inner], inner contiguous.  The 256 threads form a (ty, tx) tile with
// tx_n = 2^tx_shift lanes along the columns (each owning VEC adjacent columns) and ty_n = 256 / tx_n
// lanes along the reduced axis, combined through LDS in fixed order.  grid = outer * col_tiles *
// splits; with splits > 1 partials are stored as [split][output] (coalesced) and the last
// workgroup of a column tile to finish folds that tile's partials, split 0 first.

// Loops over a thread's columns run over all VEC of them with a predicate.  A loop with the
// run-time bound `ncol` indexes the accumulator array dynamically; the compiler then moves the
// array to LDS and, to find each thread's slot, reads the workgroup size from the dispatch packet,
// which sits in host memory: 2-10 us before the first load (measured on the arg-max kernel).
#define ZENU_FOR_COLS(j) _Pragma("unroll") for (int j = 0; j < VEC; j++) if (j < ncol)

template <typename T, typename Tr, int VEC, bool NT, bool PRE = false>
__global__ __launch_bounds__(kBlock) void reduce_cols_kernel(RedParams<T> p, uint32_t col_tiles, int tx_shift, int grid3d)
{
    typedef typename Tr::Acc A;
    __shared__ A lds[kBlock * VEC];
    const int tx_n = 1 << tx_shift;
    const int ty_n = kBlock >> tx_shift;
    const int tx = threadIdx.x & (tx_n - 1);
    const int ty = threadIdx.x >> tx_shift;
    // column tile fastest: workgroups that are dispatched together read adjacent pieces of the
    // same source rows.  The grid is (column tiles, splits, outer) when that fits the grid limits:
    // every workgroup of a launch starts at the same time, so a chain of integer divisions at the
    // top of the kernel delays the whole launch; otherwise linear (below 2^31), in 32 bits.
    uint32_t ct, split_u, q_u;
    if (grid3d) {
        ct = blockIdx.x;
        split_u = blockIdx.y;
        q_u = blockIdx.z;
    } else {
        uint32_t blk = blockIdx.x;
        const uint32_t b1 = blk / col_tiles;
        ct = blk - b1 * col_tiles;
        q_u = b1 / (uint32_t)p.splits;
        split_u = b1 - q_u * (uint32_t)p.splits;
    }
    const int split = (int)split_u;
    const int64_t q = q_u;
    const int64_t group = q * col_tiles + ct;   // the workgroups that share these outputs
    const int64_t c = ((int64_t)ct * tx_n + tx) * VEC;

    const int ncol = (c + VEC <= p.inner) ? VEC : (c < p.inner ? (int)(p.inner - c) : 0);
    const T *src = p.in + q * p.outer_stride + c;
    constexpr int U = 4;
    const int64_t R = p.R;

    // combine the ty lanes in fixed order: afterwards the row lane ty == 0 holds the result
    auto combine_rows = [&](A (&acc)[VEC]) {
        if (ty_n > 1) {
            __syncthreads();
#pragma unroll
            for (int j = 0; j < VEC; j++) lds[j * kBlock + threadIdx.x] = acc[j];   // [vector element][thread]: consecutive lanes, consecutive banks
            __syncthreads();
            int left = ty_n;
            if (ty_n > 8) {
                // more than eight row lanes (narrow column tiles): row lanes 0..7 first take every
                // eighth lane each, so that the chain of dependent LDS round trips is ty_n / 8 + 6 long
                // instead of ty_n - 1
                if (ty < 8) {
                    for (int w = ty + 8; w < ty_n; w += 8) {
#pragma unroll
                        for (int j = 0; j < VEC; j++) acc[j] = Tr::merge(acc[j], lds[j * kBlock + w * tx_n + tx]);
                    }
                }
                __syncthreads();
                if (ty < 8) {
#pragma unroll
                    for (int j = 0; j < VEC; j++) lds[j * kBlock + threadIdx.x] = acc[j];
                }
                __syncthreads();
                left = 8;
            }
            if (ty == 0) {   // row lane by row lane, the VEC columns side by side: dependent LDS round trips, but not VEC times as many
                for (int w = 1; w < left; w++) {
#pragma unroll
                    for (int j = 0; j < VEC; j++) acc[j] = Tr::merge(acc[j], lds[j * kBlock + w * tx_n + tx]);
                }
            }
        }
    };

    // the partial result of split `split` for this workgroup's columns (valid where ty == 0)
    auto partial_of = [&](int split, A (&acc)[VEC]) {
#pragma unroll
        for (int j = 0; j < VEC; j++) acc[j] = Tr::identity();
        // the splits interleave in chunks of U * ty_n source rows: all workgroups of a launch sweep
        // the source top to bottom together
        const int64_t chunk = U * ty_n;
        const int64_t row_step = (int64_t)ty_n * p.elem_stride;
        if (ncol == VEC && VEC > 1) {
            const T *ptr = src + ((int64_t)split * chunk + ty) * p.elem_stride;
            const int64_t ptr_step = (int64_t)p.splits * chunk * p.elem_stride;
            for (int64_t b = split * chunk; b < R; b += p.splits * chunk, ptr += ptr_step) {
                const int64_t r = b + ty;
                if (b + chunk <= R) {
                    Pack<T, VEC> x[U];
#pragma unroll
                    for (int u = 0; u < U; u++) x[u] = load_src<T, VEC, NT, PRE>(p, ptr + u * row_step);
#pragma unroll
                    for (int u = 0; u < U; u++) {
#pragma unroll
                        for (int j = 0; j < VEC; j++) acc[j] = Tr::update(acc[j], x[u].v[j], r + u * ty_n);
                    }
                } else {
                    const T *pt = ptr;
                    for (int64_t rr = r; rr < R; rr += ty_n, pt += row_step) {
                        Pack<T, VEC> x = load_src<T, VEC, false, PRE>(p, pt);
#pragma unroll
                        for (int j = 0; j < VEC; j++) acc[j] = Tr::update(acc[j], x.v[j], rr);
                    }
                }
            }
        } else if (ncol > 0) {
            for (int64_t b = split * chunk; b < R; b += p.splits * chunk)
                for (int64_t r = b + ty; r < R && r < b + chunk; r += ty_n)
                    ZENU_FOR_COLS(j) acc[j] = Tr::update(acc[j], src[r * p.elem_stride + j], r);
        }
        if (split == 0 && ty == 0)
            ZENU_FOR_COLS(j) acc[j] = Tr::first(acc[j], src[j]);
        combine_rows(acc);
    };

    A acc[VEC];
    partial_of(split, acc);
    const int64_t o0 = q * p.inner + c;
    if (p.splits == 1) {
        if (ty == 0)
            ZENU_FOR_COLS(j) emit_final<T, Tr>(p, o0 + j, acc[j]);
        return;
    }
    if (ty == 0)
        ZENU_FOR_COLS(j) emit_partial<T, Tr>(p, (int64_t)split * p.nout + o0 + j, acc[j]);
    if (!arrive_last(p.counters + group * p.cstride, split, p.splits, p.fan)) return;
    // fold this column tile: row lane ty takes splits ty, ty + ty_n, ...; then the fixed LDS order
#pragma unroll
    for (int j = 0; j < VEC; j++) acc[j] = Tr::identity();
    for (int s0 = ty; s0 < p.splits; s0 += 8 * ty_n) {
        A t[8][VEC];
#pragma unroll
        for (int u = 0; u < 8; u++) {       // issue the loads together, merge in split order
            const int sidx = s0 + u * ty_n;
#pragma unroll
            for (int j = 0; j < VEC; j++)
                t[u][j] = (sidx < p.splits && j < ncol) ? load_partial<T, Tr>(p, (int64_t)sidx * p.nout + o0 + j)
                                                        : Tr::identity();
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
#pragma unroll
            for (int j = 0; j < VEC; j++) acc[j] = Tr::merge(acc[j], t[u][j]);
        }
    }
    combine_rows(acc);
    if (ty == 0)
        ZENU_FOR_COLS(j) emit_final<T, Tr>(p, o0 + j, acc[j]);
    if (threadIdx.x == 0) store_agent(p.counters + group * p.cstride, 0);
}

// ---- kernel B, regular geometry ----------------------------------------------------------------------------
// Kernel B for the shape it mostly runs on -- vector columns, every column tile full (inner a
// multiple of 32 vectors), the reduced axis split over workgroups, a 3-d grid, a flat arrival
// counter -- with everything that cannot happen there taken out of the instruction stream: no
// per-column predicates, one 128-bit LDS exchange per thread instead of one per column, partials
// stored and loaded as whole vectors' worth of device-scope words without a branch each.  The
// accumulation order, the order of the LDS combine and the order of the fold are kernel B's, so
// both give the same bits.
template <typename T, typename Tr, int VEC, bool NT, bool PRE = false, int U = 4>
__global__ __launch_bounds__(kBlock) void reduce_cols_regular_kernel(RedParams<T> p)
{
    typedef typename Tr::Acc A;
    struct Cols {
        A a[VEC];
    };
    __shared__ Cols lds[kBlock];
    constexpr int TX = 32, TY = kBlock / TX;
    const int tx = threadIdx.x & (TX - 1), ty = threadIdx.x / TX;
    const int split = (int)blockIdx.y, splits = p.splits;
    const int64_t q = blockIdx.z;
    const int64_t c = ((int64_t)blockIdx.x * TX + tx) * VEC;
    const T *src = p.in + q * p.outer_stride + c;
    const int64_t R = p.R, es = p.elem_stride;

    // afterwards the row lane ty == 0 holds the result of the TY lanes, merged in lane order
    auto combine_rows = [&](Cols &acc) {
        __syncthreads();
        lds[threadIdx.x] = acc;
        __syncthreads();
        if (ty == 0) {
#pragma unroll
            for (int w = 1; w < TY; w++) {
                const Cols o = lds[w * TX + tx];
#pragma unroll
                for (int j = 0; j < VEC; j++) acc.a[j] = Tr::merge(acc.a[j], o.a[j]);
            }
        }
    };

    Cols acc;
#pragma unroll
    for (int j = 0; j < VEC; j++) acc.a[j] = Tr::identity();
    constexpr int chunk = U * TY;
    for (int64_t b = (int64_t)split * chunk; b < R; b += (int64_t)splits * chunk) {
        const int64_t r = b + ty;
        if (b + chunk <= R) {
            Pack<T, VEC> x[U];
#pragma unroll
            for (int u = 0; u < U; u++) x[u] = load_src<T, VEC, NT, PRE>(p, src + (r + u * TY) * es);
#pragma unroll
            for (int u = 0; u < U; u++) {
#pragma unroll
                for (int j = 0; j < VEC; j++) acc.a[j] = Tr::update(acc.a[j], x[u].v[j], r + u * TY);
            }
        } else {
            for (int64_t rr = r; rr < R; rr += TY) {
                const Pack<T, VEC> x = load_src<T, VEC, false, PRE>(p, src + rr * es);
#pragma unroll
                for (int j = 0; j < VEC; j++) acc.a[j] = Tr::update(acc.a[j], x.v[j], rr);
            }
        }
    }
    if (split == 0 && ty == 0) {
#pragma unroll
        for (int j = 0; j < VEC; j++) acc.a[j] = Tr::first(acc.a[j], src[j]);
    }
    combine_rows(acc);

    const int64_t o0 = q * p.inner + c;
    if (ty == 0) {
#pragma unroll
        for (int j = 0; j < VEC; j++) emit_partial<T, Tr>(p, (int64_t)split * p.nout + o0 + j, acc.a[j]);
    }
    const int64_t group = q * gridDim.x + blockIdx.x;
    if (!arrive_last(p.counters + group, split, splits, splits)) return;
    // fold this column tile: row lane ty takes splits ty, ty + TY, ... two at a time, then the LDS order
#pragma unroll
    for (int j = 0; j < VEC; j++) acc.a[j] = Tr::identity();
    for (int s0 = ty; s0 < splits; s0 += 2 * TY) {
        A t[2][VEC];
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const int sidx = s0 + u * TY;
            if (sidx < splits) {
#pragma unroll
                for (int j = 0; j < VEC; j++) t[u][j] = load_partial<T, Tr>(p, (int64_t)sidx * p.nout + o0 + j);
            } else {
#pragma unroll
                for (int j = 0; j < VEC; j++) t[u][j] = Tr::identity();
            }
        }
#pragma unroll
        for (int u = 0; u < 2; u++) {
#pragma unroll
            for (int j = 0; j < VEC; j++) acc.a[j] = Tr::merge(acc.a[j], t[u][j]);
        }
    }
    combine_rows(acc);
    if (ty == 0) {
        if constexpr (!Tr::kHasIdx) {
            Pack<T, VEC> r;
#pragma unroll
            for (int j = 0; j < VEC; j++) r.v[j] = Tr::key(acc.a[j]);
            store_pack<T, VEC, false>(p.out_val + o0, r);
        } else {
#pragma unroll
            for (int j = 0; j < VEC; j++) emit_final<T, Tr>(p, o0 + j, acc.a[j]);
        }
    }
    if (threadIdx.x == 0) store_agent(p.counters + group, 0);
}

// ---- host side ---------------------------------------------------------------------------------------------

// the source is read once; when it is larger than the caches the loads carry the streaming hint
template <typename T> inline bool stream_source(const RedParams<T> &p)
{
    return p.nout * p.R * (int64_t)sizeof(T) >= kStreamBytes;
}

template <typename T, typename Tr>
int launch_rows(const RedParams<T> &p, hipStream_t s)
{
    constexpr int VEC = VecOf<T>::N;
    const bool vec = p.elem_stride == 1 && p.inner == 1 && aligned16(p.in) && p.outer_stride % VEC == 0;
    const bool nt = vec && stream_source(p);
    const bool wave_row = p.splits == 1 && p.R <= 1024;
    if (wave_row) {
        int64_t grid = (p.nout + kWaves - 1) / kWaves;
        if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
        if (nt)       reduce_rows_kernel<T, Tr, VEC, kWaveRow, true, kRowsU><<<(unsigned)grid, kBlock, 0, s>>>(p);
        else if (vec) reduce_rows_kernel<T, Tr, VEC, kWaveRow, false, kRowsU><<<(unsigned)grid, kBlock, 0, s>>>(p);
        else          reduce_rows_kernel<T, Tr, 1, kWaveRow, false, kRowsU><<<(unsigned)grid, kBlock, 0, s>>>(p);
    } else {
        int64_t grid = p.nout * p.splits;
        if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
        if (p.splits > 1) {
            if (p.nout > 65535) return ZENU_ERR_UNSUPPORTED;   // never: rows are split only when there are few of them
            const dim3 g((unsigned)p.splits, (unsigned)p.nout);
            if (nt)       reduce_rows_kernel<T, Tr, VEC, kSplitRow, true, kSplitU><<<g, kBlock, 0, s>>>(p);
            else if (vec) reduce_rows_kernel<T, Tr, VEC, kSplitRow, false, kRowsU><<<g, kBlock, 0, s>>>(p);
            else          reduce_rows_kernel<T, Tr, 1, kSplitRow, false, kRowsU><<<g, kBlock, 0, s>>>(p);
        } else {
            if (nt)       reduce_rows_kernel<T, Tr, VEC, kBlockRow, true, kRowsU><<<(unsigned)grid, kBlock, 0, s>>>(p);
            else if (vec) reduce_rows_kernel<T, Tr, VEC, kBlockRow, false, kRowsU><<<(unsigned)grid, kBlock, 0, s>>>(p);
            else          reduce_rows_kernel<T, Tr, 1, kBlockRow, false, kRowsU><<<(unsigned)grid, kBlock, 0, s>>>(p);
        }
    }
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

// threads along the columns for a cols launch: a power of two covering the row, at most kColsTx
constexpr int64_t kSmallColsRows = 512, kSmallColsBytes = 4 << 20;   // see reduce_strided
constexpr int kColsTx = 32;  // 32 lanes x 16 B = 512 B of a source row per wavefront half (measured best of 8..256)
inline int cols_tx_shift(int64_t inner, int v)
{
    const int64_t vcols = (inner + v - 1) / v;
    int shift = 0;
    while ((1 << shift) < kColsTx && ((int64_t)1 << shift) < vcols) shift++;
    return shift;
}

template <typename T> inline bool cols_vec_ok(const RedParams<T> &p)
{
    constexpr int VEC = VecOf<T>::N;
    return aligned16(p.in) && p.inner % VEC == 0 && p.outer_stride % VEC == 0 && p.elem_stride % VEC == 0;
}

template <typename T, typename Tr>
int launch_cols(const RedParams<T> &p, hipStream_t s)
{
    constexpr int VEC = VecOf<T>::N;
    const bool vec = cols_vec_ok(p);
    const bool nt = vec && stream_source(p);
    const int v = vec ? VEC : 1;
    const int shift = p.cols_shift;
    const int64_t per_tile = ((int64_t)1 << shift) * v;
    const int64_t col_tiles = (p.inner + per_tile - 1) / per_tile;
    const int64_t outer = p.nout / p.inner;
    int64_t grid = outer * col_tiles * p.splits;
    if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
    const int g3 = (p.splits <= 65535 && outer <= 65535) ? 1 : 0;
    const dim3 g = g3 ? dim3((unsigned)col_tiles, (unsigned)p.splits, (unsigned)outer) : dim3((unsigned)grid);
    const uint32_t ctl = (uint32_t)col_tiles;
    // the regular geometry: full vector tiles of 32 x 8 threads, a split axis with a flat counter
    const bool regular = vec && g3 && shift == 5 && p.inner % per_tile == 0 && p.splits > 1 && p.fan >= p.splits &&
                         p.cstride == 1 && (Tr::kHasIdx || aligned16(p.out_val));
    if constexpr (!Tr::kHasIdx && std::is_same<Tr, SumTr<T>>::value) {
        if (p.pre_x) {   // the transform rides on the vector paths only (the caller has checked the layout)
            if (!vec) return ZENU_ERR_UNSUPPORTED;
            if (regular) {
                if (nt) reduce_cols_regular_kernel<T, Tr, VEC, true, true><<<g, kBlock, 0, s>>>(p);
                else    reduce_cols_regular_kernel<T, Tr, VEC, false, true><<<g, kBlock, 0, s>>>(p);
            } else {
                if (nt) reduce_cols_kernel<T, Tr, VEC, true, true><<<g, kBlock, 0, s>>>(p, ctl, shift, g3);
                else    reduce_cols_kernel<T, Tr, VEC, false, true><<<g, kBlock, 0, s>>>(p, ctl, shift, g3);
            }
            ZENU_LAUNCH_CHECK();
            return ZENU_OK;
        }
    }
    if (regular) {
        if (nt) reduce_cols_regular_kernel<T, Tr, VEC, true><<<g, kBlock, 0, s>>>(p);
        else    reduce_cols_regular_kernel<T, Tr, VEC, false><<<g, kBlock, 0, s>>>(p);
        ZENU_LAUNCH_CHECK();
        return ZENU_OK;
    }
    if (nt)       reduce_cols_kernel<T, Tr, VEC, true><<<g, kBlock, 0, s>>>(p, ctl, shift, g3);
    else if (vec) reduce_cols_kernel<T, Tr, VEC, false><<<g, kBlock, 0, s>>>(p, ctl, shift, g3);
    else          reduce_cols_kernel<T, Tr, 1, false><<<g, kBlock, 0, s>>>(p, ctl, shift, g3);
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

// Reduce a source addressed as src[q * outer_stride + c + r * elem_stride] (q < outer, c < inner,
// r < R; the inner run has unit stride) into contiguous outputs of outer*inner elements.
template <typename T, typename Tr>
int reduce_strided(const T *src, int64_t outer, int64_t R, int64_t inner, int64_t outer_stride,
                   int64_t elem_stride, T *out_val, int64_t *out_idx, hipStream_t s,
                   const FixedScratch *fixed = nullptr, const T *pre_x = nullptr, T *pre_out = nullptr,
                   T pre_alpha = (T)0)
{
    constexpr int VEC = VecOf<T>::N;
    const int64_t nout = outer * inner;
    if (nout == 0) return ZENU_OK;
    if (R <= 0) {
        // an empty axis: sums are zero (sum.rs:18-25 adds nothing to zeros, BLAS asum of n = 0 is 0);
        // the arg-max scan reads element 0 (max.rs:22) -- an error, as in the reference
        if (Tr::kHasIdx) return ZENU_ERR_SHAPE;
        return zenu_hip_memset_zero(out_val, (size_t)nout * sizeof(T), reinterpret_cast<zenu_stream_t>(s));
    }
    if (Tr::kHasIdx && R >= kNoIdx) return ZENU_ERR_UNSUPPORTED;  // positions are tracked in 32 bits
    // workgroups to aim for when the outputs alone do not fill the GPU: two per CU.  More splits
    // shorten the streaming phase but lengthen the serial hand-off at the end (measured 1..16).
    const int64_t target_blocks = (int64_t)device_info().num_cus * 2;

    RedParams<T> p;
    p.in = src;
    p.nout = nout;
    p.R = R;
    p.inner = inner;
    p.outer_stride = outer_stride;
    p.elem_stride = elem_stride;
    p.out_val = out_val;
    p.out_idx = out_idx;
    p.part_key = nullptr;
    p.part_idx = nullptr;
    p.counters = nullptr;
    p.fan = 1;
    p.cstride = 1;
    p.slots = nullptr;
    p.epoch = 0;
    p.spin_limit = 0;
    p.fallbacks = g_fold_fallbacks_ptr;
    p.pre_x = pre_x;
    p.pre_out = pre_out;
    p.pre_alpha = pre_alpha;
    p.gsrc = src;
    p.g_outer_stride = outer_stride;
    p.g_elem_stride = elem_stride;

    const bool use_cols = inner >= 16;
    if (pre_x && (!use_cols || !cols_vec_ok(p))) return ZENU_ERR_UNSUPPORTED;   // the caller falls back to two launches
    int64_t splits = 1, groups = nout;
    p.cols_shift = 0;
    if (use_cols) {
        const int v = cols_vec_ok(p) ? VEC : 1;
        int shift = cols_tx_shift(inner, v);
        auto tiles_at = [&](int sh) { return (inner + (((int64_t)1 << sh) * v) - 1) / (((int64_t)1 << sh) * v); };
        // A small source with a short reduced axis is bound by latencies, and the hand-off of a split
        // (about 3 us) is the longest of them: narrower column tiles (down to 64-byte row pieces, which
        // stream at less than half the rate, but there is little to stream) give more workgroups
        // without one.  Column sums of [256,512] f32 with the ReLU-gradient transform: 7.7 us as
        // 4 tiles x 4 splits, 5.8 us as 16 tiles of 32 columns, 5.0 us as 32 tiles of 16 columns.
        if (v > 1 && R <= kSmallColsRows && outer * R * inner * (int64_t)sizeof(T) <= kSmallColsBytes)
            while (shift > 2 && outer * tiles_at(shift) < target_blocks) shift--;
        p.cols_shift = shift;
        const int64_t col_tiles = tiles_at(shift);
        const int64_t ty_n = kBlock >> shift;
        groups = outer * col_tiles;
        if (groups < target_blocks) {
            splits = (target_blocks + groups - 1) / groups;
            const int64_t max_splits = (R + 8 * ty_n - 1) / (8 * ty_n);  // >= 8 rows per thread
            if (splits > max_splits) splits = max_splits;
        }
    } else {
        if (nout < target_blocks) {
            splits = (target_blocks + nout - 1) / nout;
            const int64_t per_block = (int64_t)kBlock * VEC * 8;  // keep >= 8 vectors per lane
            const int64_t max_splits = (R + per_block - 1) / per_block;
            if (splits > max_splits) splits = max_splits;
        }
    }
    if (splits < 1) splits = 1;
    if (splits > 4096) splits = 4096;
    p.splits = (int)splits;

    if (splits == 1) return use_cols ? launch_cols<T, Tr>(p, s) : launch_rows<T, Tr>(p, s);

    // one launch: partials in a workspace, folded by the last workgroup of each group to arrive
    // arrival tree: eight splits per leaf once a flat counter would serialise
    int fan = (int)splits, cstride = 1;
    if (splits > 16) {
        fan = 8;   // measured on 512 splits: 2 / 4 / 8 / 16 / 23 (= sqrt) / 64 / flat -> 23.6 / 22.9 / 22.8 / 23.4 / 24.3 / 25.0 / 25.0 us
        cstride = 1 + (int)((splits + fan - 1) / fan);
    }
    const size_t key_bytes = ((size_t)nout * splits * sizeof(T) + 255) / 256 * 256;
    const size_t idx_bytes = Tr::kHasIdx ? (size_t)nout * splits * sizeof(int32_t) : 0;
    if (!fixed && !use_cols) {
        // Tagged words from the stream's ring when the launch may use them (not while the stream
        // records a graph, not beyond half the ring).  Rows only: with the column kernel's many
        // groups the polls of one group queue behind the streaming of the others and the counters
        // are faster (sum over axis 0 of [8192,4096] f32: 24.3 us against 25.1 us; of
        // [131072,256]: 32 us against 49 us), while split rows gain 0.3 - 1.2 us.
        uint32_t epoch = 0;
        uint64_t *slots = reserve_slots(nout * splits * SlotWords<T, Tr>::W, s, &epoch);
        if (slots) {
            // The request the counter path would make, once per stream and size: it leaves a block of
            // that size in the pool of this stream, so that a later capture of the same call (which
            // takes the counter path) finds it there and does not have to go to the driver.
            if (rehearsal_needed(key_bytes + idx_bytes, s)) {
                Workspace rehearse(key_bytes + idx_bytes, s);
                if (rehearse.status) return rehearse.status;
            }
            p.slots = slots;
            p.epoch = epoch;
            p.spin_limit = reduce_spin_limit();
            return launch_rows<T, Tr>(p, s);
        }
    }
    if (fixed) {
        // the caller may not allocate: counters and partials live in the static scratch, which
        // every such call on the device shares and which keeps the last call's contents
        if (groups * cstride > fixed->n_counters) {
            fan = (int)splits;
            cstride = 1;
        }
        if (groups * cstride > fixed->n_counters || key_bytes + idx_bytes > fixed->partial_bytes)
            return ZENU_ERR_SCRATCH_LIMIT;
        // counters must start at zero; a fill kernel, not a memset node, so the call can be captured
        int rc = zenu_hip_memset_zero(fixed->counters, (size_t)(groups * cstride) * sizeof(int),
                                      reinterpret_cast<zenu_stream_t>(s));
        if (rc) return rc;
        p.fan = fan;
        p.cstride = cstride;
        p.part_key = static_cast<T *>(fixed->partials);
        p.part_idx = Tr::kHasIdx ? reinterpret_cast<int32_t *>(static_cast<char *>(fixed->partials) + key_bytes) : nullptr;
        p.counters = fixed->counters;
        return use_cols ? launch_cols<T, Tr>(p, s) : launch_rows<T, Tr>(p, s);
    }
    int *counters = reserve_counters(groups * cstride, s);
    if (!counters && cstride > 1) {   // too many groups for trees: flat counters
        fan = (int)splits;
        cstride = 1;
        counters = reserve_counters(groups, s);
    }
    if (!counters) return ZENU_ERR_UNSUPPORTED;
    p.fan = fan;
    p.cstride = cstride;
    Workspace ws(key_bytes + idx_bytes, s);
    if (ws.status) return ws.status;
    p.part_key = static_cast<T *>(ws.ptr);
    p.part_idx = Tr::kHasIdx ? reinterpret_cast<int32_t *>(static_cast<char *>(ws.ptr) + key_bytes) : nullptr;
    p.counters = counters;
    return use_cols ? launch_cols<T, Tr>(p, s) : launch_rows<T, Tr>(p, s);
}

// a contiguous [outer, R, inner] source
template <typename T, typename Tr>
int reduce_contiguous(const T *src, int64_t outer, int64_t R, int64_t inner, T *out_val,
                      int64_t *out_idx, hipStream_t s)
{
    return reduce_strided<T, Tr>(src, outer, R, inner, R * inner, inner, out_val, out_idx, s);
}

}  // namespace

namespace {

// ---- tensor-level wrappers ------------------------------------------------------------------------------------

// out must hold src's shape minus `axis`, or with that axis kept as 1 (keep_dim)
bool reduced_shape_ok(const zenu_tensor_t &out, const zenu_tensor_t &src, int axis)
{
    if (out.ndim == src.ndim - 1) {
        int k = 0;
        for (int i = 0; i < src.ndim; i++) {
            if (i == axis) continue;
            if (out.shape[k++] != src.shape[i]) return false;
        }
        return true;
    }
    if (out.ndim == src.ndim) {
        for (int i = 0; i < src.ndim; i++)
            if (out.shape[i] != (i == axis ? 1 : src.shape[i])) return false;
        return true;
    }
    return false;
}

enum RedKind { kSum, kAsum, kMax };

struct StridedMap {
    bool ok;
    int64_t outer, inner, outer_stride, elem_stride;
};

// kept dims of `src` (every dim but `axis`, in order) as [outer with a uniform stride chain] x
// [inner unit-stride run]; size-1 dims never matter
StridedMap map_strided(const zenu_tensor_t &src, int axis)
{
    StridedMap m = {false, 1, 1, 0, src.stride[axis]};
    int64_t shape[kMaxDim], stride[kMaxDim];
    int k = 0;
    for (int i = 0; i < src.ndim; i++) {
        if (i == axis || src.shape[i] == 1) continue;
        if (src.shape[i] == 0 || src.stride[i] <= 0) return m;
        shape[k] = src.shape[i];
        stride[k] = src.stride[i];
        k++;
    }
    if (src.shape[axis] > 1 && src.stride[axis] <= 0) return m;
    // trailing unit-stride run
    int j = k;
    int64_t run = 1;
    while (j > 0 && stride[j - 1] == run) {
        run *= shape[j - 1];
        j--;
    }
    m.inner = run;
    // the rest must chain: stride[i] == stride[i+1] * shape[i+1]
    for (int i = 0; i + 1 < j; i++)
        if (stride[i] != stride[i + 1] * shape[i + 1]) return m;
    for (int i = 0; i < j; i++) m.outer *= shape[i];
    m.outer_stride = j > 0 ? stride[j - 1] : 0;
    // the reduced elements of one output must not run into the next output's inner run or the
    // kernel's vector paths would mis-assume; plain strided addressing needs no further condition
    m.ok = true;
    return m;
}

template <typename T>
int reduce_axis_t(int kind, int dtype, const zenu_tensor_t *out, int64_t *out_idx,
                  const zenu_tensor_t &src, int axis, hipStream_t s, const FixedScratch *fixed = nullptr)
{
    const int64_t n = num_elm(src);
    int64_t outer = 1, inner = 1;
    for (int i = 0; i < axis; i++) outer *= src.shape[i];
    for (int i = axis + 1; i < src.ndim; i++) inner *= src.shape[i];
    const int64_t R = src.shape[axis];
    const int64_t nout = outer * inner;

    // A view is reduced in place when its kept dims, in output order, split into a leading group
    // with one uniform stride chain (the kernel's `outer`) and a trailing group that is a unit-stride
    // run (the kernel's `inner`): transposed matrices, row slices, index_axis views.  Anything
    // else goes through a contiguous copy first (to_default_stride, as max.rs:49 does).
    StridedMap map = map_strided(src, axis);
    const T *sp = static_cast<const T *>(src.ptr);
    if (fixed && !map.ok) return ZENU_ERR_UNSUPPORTED;   // would need a copy of the whole source
    Workspace wsrc(map.ok ? 0 : (size_t)n * sizeof(T), s);
    if (!map.ok) {
        if (wsrc.status) return wsrc.status;
        zenu_tensor_t tmp = default_view(wsrc.ptr, src.ndim, src.shape);
        int rc = zenu_hip_copy(dtype, &tmp, &src, s);
        if (rc) return rc;
        sp = static_cast<const T *>(wsrc.ptr);
        map.outer = outer;
        map.inner = inner;
        map.outer_stride = R * inner;
        map.elem_stride = inner;
    }

    // contiguous destination, or a temporary that is copied out afterwards
    T *ov = nullptr;
    bool need_copy = false;
    const bool stage_out = out && !is_default_stride_strict(*out);
    if (fixed && stage_out && (size_t)nout * sizeof(T) > fixed->stage_bytes) return ZENU_ERR_SCRATCH_LIMIT;
    Workspace wout((stage_out && !fixed) ? (size_t)(nout ? nout : 1) * sizeof(T) : 0, s);
    if (out) {
        if (!stage_out) {
            ov = static_cast<T *>(out->ptr);
        } else if (fixed) {
            ov = static_cast<T *>(fixed->stage);
            need_copy = true;
        } else {
            if (wout.status) return wout.status;
            ov = static_cast<T *>(wout.ptr);
            need_copy = true;
        }
    }
    int rc;
    if (kind == kSum) rc = reduce_strided<T, SumTr<T>>(sp, map.outer, R, map.inner, map.outer_stride, map.elem_stride, ov, nullptr, s, fixed);
    else if (kind == kAsum) rc = reduce_strided<T, AsumTr<T>>(sp, map.outer, R, map.inner, map.outer_stride, map.elem_stride, ov, nullptr, s, fixed);
    else rc = reduce_strided<T, ArgmaxTr<T>>(sp, map.outer, R, map.inner, map.outer_stride, map.elem_stride, ov, out_idx, s, fixed);
    if (rc) return rc;
    if (need_copy) {
        zenu_tensor_t tmp = default_view(ov, out->ndim, out->shape);
        rc = zenu_hip_copy(dtype, out, &tmp, s);
    }
    return rc;
}

int reduce_axis(int kind, int dtype, const zenu_tensor_t *out, int64_t *out_idx, const zenu_tensor_t *src,
                int axis, hipStream_t s, const FixedScratch *fixed = nullptr)
{
    int rc = validate_tensor(src);
    if (!rc && out) rc = validate_tensor(out);
    if (!rc) rc = fixed ? ZENU_OK : ensure_init();   // the allocation-free caller has checked that init ran
    if (rc) return rc;
    if (axis < 0 || axis >= src->ndim) return ZENU_ERR_AXIS;
    if (out && !reduced_shape_ok(*out, *src, axis)) return ZENU_ERR_SHAPE;
    {   // results that share memory with the source would be read back as input by other workgroups
        const size_t esz = dtype == ZENU_F64 ? 8 : 4;
        int64_t nout = 1;
        for (int i = 0; i < src->ndim; i++)
            if (i != axis) nout *= src->shape[i];
        if (out && src->shape[axis] > 1 && check_output_alias(*out, *src, esz)) return ZENU_ERR_ARG;
        if (out_idx && view_overlaps(*src, esz, out_idx, (size_t)nout * sizeof(int64_t))) return ZENU_ERR_ARG;
    }
    if (dtype == ZENU_F32) return reduce_axis_t<float>(kind, dtype, out, out_idx, *src, axis, s, fixed);
    if (dtype == ZENU_F64) return reduce_axis_t<double>(kind, dtype, out, out_idx, *src, axis, s, fixed);
    return ZENU_ERR_ARG;
}

// whole-tensor reductions: view the (contiguous copy of the) source as one row
int reduce_all(int kind, int dtype, void *out_val, int64_t *out_idx, const zenu_tensor_t *src, hipStream_t s)
{
    int rc = validate_tensor(src);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    const int64_t n = num_elm(*src);
    const size_t esz = dtype == ZENU_F32 ? 4 : 8;
    if (dtype != ZENU_F32 && dtype != ZENU_F64) return ZENU_ERR_ARG;
    if (n > 1 && ((out_val && view_overlaps(*src, esz, out_val, esz)) ||
                  (out_idx && view_overlaps(*src, esz, out_idx, sizeof(int64_t)))))
        return ZENU_ERR_ARG;   // the result would overwrite an element other workgroups still read
    if (n <= 0) {   // nothing to add: 0; nothing to take a maximum of: an error
        if (kind == kMax) return ZENU_ERR_SHAPE;
        return zenu_hip_memset_zero(out_val, esz, reinterpret_cast<zenu_stream_t>(s));
    }
    Workspace wsrc(is_default_stride_strict(*src) ? 0 : (size_t)n * esz, s);
    const void *sp = src->ptr;
    if (!is_default_stride_strict(*src)) {
        if (wsrc.status) return wsrc.status;
        zenu_tensor_t tmp = default_view(wsrc.ptr, src->ndim, src->shape);
        rc = zenu_hip_copy(dtype, &tmp, src, s);
        if (rc) return rc;
        sp = wsrc.ptr;
    }
    if (dtype == ZENU_F32) {
        const float *f = static_cast<const float *>(sp);
        float *ov = static_cast<float *>(out_val);
        if (kind == kSum) return reduce_contiguous<float, SumTr<float>>(f, 1, n, 1, ov, nullptr, s);
        if (kind == kAsum) return reduce_contiguous<float, AsumTr<float>>(f, 1, n, 1, ov, nullptr, s);
        return reduce_contiguous<float, ArgmaxTr<float>>(f, 1, n, 1, ov, out_idx, s);
    }
    const double *d = static_cast<const double *>(sp);
    double *ov = static_cast<double *>(out_val);
    if (kind == kSum) return reduce_contiguous<double, SumTr<double>>(d, 1, n, 1, ov, nullptr, s);
    if (kind == kAsum) return reduce_contiguous<double, AsumTr<double>>(d, 1, n, 1, ov, nullptr, s);
    return reduce_contiguous<double, ArgmaxTr<double>>(d, 1, n, 1, ov, out_idx, s);
}

template <typename T>
int relu_backward_bias_grad_t(const zenu_tensor_t &gx, const zenu_tensor_t &gbias, const zenu_tensor_t &gy,
                                     const zenu_tensor_t &x, double alpha, hipStream_t s)
{
    const int64_t n = gbias.shape[gbias.ndim - 1];
    const int64_t rows = num_elm(gy) / n;
    return reduce_strided<T, SumTr<T>>(static_cast<const T *>(gy.ptr), 1, rows, n, rows * n, n,
                                       static_cast<T *>(gbias.ptr), nullptr, s, nullptr,
                                       static_cast<const T *>(x.ptr), static_cast<T *>(gx.ptr), (T)alpha);
}

}  // namespace

// Called once by the library's init, with its device current: the device address of the static
// scratch.  Each device holds its own copy of the array at its own address; the library drives
// one device per process, so one pointer is kept.
int init_static_scratch()
{
    if (g_scratch_ptr) return ZENU_OK;
    void *p = nullptr;
    ZENU_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    if (!p) return ZENU_ERR_HIP;
    g_scratch_ptr = static_cast<unsigned char *>(p);
    void *f = nullptr;
    ZENU_HIP_TRY(hipGetSymbolAddress(&f, HIP_SYMBOL(fold_fallbacks)));
    if (!f) return ZENU_ERR_HIP;
    ZENU_HIP_TRY(hipMemset(f, 0, sizeof(unsigned int)));
    g_fold_fallbacks_ptr = static_cast<unsigned int *>(f);
    return ZENU_OK;
}

}  // namespace zenu

using namespace zenu;

extern "C" {

int zenu_hip_sum_axis_noalloc(int dtype, const zenu_tensor_t *out, const zenu_tensor_t *src, int axis,
                              zenu_stream_t stream)
{
    if (!out) return ZENU_ERR_ARG;
    // initialising the library allocates (pool, counter rings): not from here
    if (!library_ready() || !g_scratch_ptr) return ZENU_ERR_NOT_INIT;
    FixedScratch fx;
    fx.counters = reinterpret_cast<int *>(g_scratch_ptr);
    fx.n_counters = (int64_t)kScratchCounters;
    fx.partials = g_scratch_ptr + kScratchCounterBytes;
    fx.partial_bytes = kScratchPartialBytes;
    fx.stage = g_scratch_ptr + kScratchCounterBytes + kScratchPartialBytes;
    fx.stage_bytes = kScratchStageBytes;
    return reduce_axis(kSum, dtype, out, nullptr, src, axis, as_stream(stream), &fx);
}

int zenu_hip_reduce_fallback_count(uint64_t *count)
{
    if (!count) return ZENU_ERR_ARG;
    if (!library_ready() || !g_fold_fallbacks_ptr) return ZENU_ERR_NOT_INIT;
    unsigned int v = 0;
    ZENU_HIP_TRY(hipMemcpy(&v, g_fold_fallbacks_ptr, sizeof v, hipMemcpyDeviceToHost));   // waits for the device
    *count = v;
    return ZENU_OK;
}

int zenu_hip_sum_axis(int dtype, const zenu_tensor_t *out, const zenu_tensor_t *src, int axis,
                      zenu_stream_t stream)
{
    if (!out) return ZENU_ERR_ARG;
    return reduce_axis(kSum, dtype, out, nullptr, src, axis, as_stream(stream));
}

int zenu_hip_sum_all(int dtype, void *out_dev, const zenu_tensor_t *src, zenu_stream_t stream)
{
    if (!out_dev) return ZENU_ERR_ARG;
    return reduce_all(kSum, dtype, out_dev, nullptr, src, as_stream(stream));
}

// ShapeStride::is_contiguous (zenu-matrix/src/shape_stride.rs:65-83) on dims k.. of `t`
static bool ref_is_contiguous(const zenu_tensor_t &t, int k)
{
    const int nd = t.ndim - k;
    if (nd <= 0) return true;
    int order[kMaxDim];
    for (int i = 0; i < nd; i++) order[i] = k + i;
    for (int i = 1; i < nd; i++) {  // stable, by decreasing stride
        int o = order[i], j = i - 1;
        while (j >= 0 && t.stride[order[j]] < t.stride[o]) { order[j + 1] = order[j]; j--; }
        order[j + 1] = o;
    }
    int64_t d[kMaxDim];
    d[nd - 1] = 1;
    for (int i = nd - 2; i >= 0; i--) d[i] = d[i + 1] * t.shape[order[i + 1]];
    const int64_t s0 = t.stride[order[0]];
    if (s0 == 0 || d[0] % s0 != 0) return false;
    const int64_t n = d[0] / s0;
    for (int i = 0; i < nd; i++)
        if (d[i] * n != t.stride[order[i]]) return false;
    return true;
}

int zenu_hip_asum(int dtype, void *out_dev, const zenu_tensor_t *src, zenu_stream_t stream)
{
    if (!out_dev) return ZENU_ERR_ARG;
    int rc = validate_tensor(src);
    if (rc) return rc;
    // Matrix::asum (asum.rs:49-68) peels leading axes until the remaining view is contiguous and
    // sums |x| there; a view that never becomes contiguous bottoms out at 0-d items, which are
    // returned raw (no abs).  Same result here, in one reduction.
    if (src->ndim == 0) {
        const size_t esz = dtype == ZENU_F32 ? 4 : 8;
        return zenu_hip_memcpy_d2d(out_dev, src->ptr, esz, stream);
    }
    bool abs_sum = false;
    for (int k = 0; k < src->ndim && !abs_sum; k++) abs_sum = ref_is_contiguous(*src, k);
    return reduce_all(abs_sum ? kAsum : kSum, dtype, out_dev, nullptr, src, as_stream(stream));
}

int zenu_hip_max_axis(int dtype, const zenu_tensor_t *out, const zenu_tensor_t *src, int axis,
                      zenu_stream_t stream)
{
    if (!out) return ZENU_ERR_ARG;
    return reduce_axis(kMax, dtype, out, nullptr, src, axis, as_stream(stream));
}

int zenu_hip_max_axis_idx(int dtype, int64_t *out_idx_dev, const zenu_tensor_t *src, int axis,
                          zenu_stream_t stream)
{
    if (!out_idx_dev) return ZENU_ERR_ARG;
    return reduce_axis(kMax, dtype, nullptr, out_idx_dev, src, axis, as_stream(stream));
}

int zenu_hip_max_idx(int dtype, int64_t *out_flat_idx_dev, void *out_val_dev, const zenu_tensor_t *src,
                     zenu_stream_t stream)
{
    if (!out_flat_idx_dev && !out_val_dev) return ZENU_ERR_ARG;
    return reduce_all(kMax, dtype, out_val_dev, out_flat_idx_dev, src, as_stream(stream));
}

int zenu_hip_relu_backward_bias_grad(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gbias,
                                     const zenu_tensor_t *gy, const zenu_tensor_t *x, double alpha,
                                     zenu_stream_t stream)
{
    int rc = validate_tensor(gx);
    if (!rc) rc = validate_tensor(gbias);
    if (!rc) rc = validate_tensor(gy);
    if (!rc) rc = validate_tensor(x);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (dtype != ZENU_F32 && dtype != ZENU_F64) return ZENU_ERR_ARG;
    if (!same_shape(*gx, *gy) || !same_shape(*gx, *x)) return ZENU_ERR_SHAPE;
    const size_t esz = dtype == ZENU_F32 ? 4 : 8;
    if (view_overlaps(*gx, esz, gbias->ptr, (size_t)num_elm(*gbias) * esz) ||
        view_overlaps(*gy, esz, gbias->ptr, (size_t)num_elm(*gbias) * esz) ||
        view_overlaps(*x, esz, gbias->ptr, (size_t)num_elm(*gbias) * esz) || check_output_alias(*gx, *x, esz))
        return ZENU_ERR_ARG;
    // one launch when the gradient is a whole [.., N] tensor and the bias gradient its [N] (or [1, .., N])
    // column sums; anything else is the two calls it stands for
    bool fused = gx->ndim >= 2 && gbias->ndim >= 1 && num_elm(*gy) > 0 && is_default_stride_strict(*gx) &&
                 is_default_stride_strict(*gy) && is_default_stride_strict(*x) && is_default_stride_strict(*gbias) &&
                 aligned16(gx->ptr) && aligned16(x->ptr) && aligned16(gy->ptr);
    if (fused) {
        const int64_t n = gx->shape[gx->ndim - 1];
        fused = gbias->shape[gbias->ndim - 1] == n && num_elm(*gbias) == n;
    }
    if (fused) {
        rc = dtype == ZENU_F32 ? relu_backward_bias_grad_t<float>(*gx, *gbias, *gy, *x, alpha, as_stream(stream))
                               : relu_backward_bias_grad_t<double>(*gx, *gbias, *gy, *x, alpha, as_stream(stream));
        if (rc != ZENU_ERR_UNSUPPORTED) return rc;
    }
    rc = zenu_hip_relu_backward(dtype, gx, gy, x, alpha, stream);
    if (rc) return rc;
    return zenu_hip_sum_to(dtype, gbias, gx, stream);
}

int zenu_hip_sum_to(int dtype, const zenu_tensor_t *target, const zenu_tensor_t *src, zenu_stream_t stream)
{
    // sum.rs:35-94
    int rc = validate_tensor(src);
    if (!rc) rc = validate_tensor(target);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (dtype != ZENU_F32 && dtype != ZENU_F64) return ZENU_ERR_ARG;
    if (src->ndim < target->ndim) return ZENU_ERR_RANK;
    hipStream_t s = as_stream(stream);
    if (same_shape(*src, *target)) return zenu_hip_copy(dtype, target, src, stream);
    const size_t esz = dtype == ZENU_F32 ? 4 : 8;
    const int diff = src->ndim - target->ndim;

    // list of axes to reduce, in the order the reference reduces them
    int axes[kMaxDim * 2], keep[kMaxDim * 2], na = 0;
    if (diff == 0) {
        for (int i = 0; i < src->ndim; i++) {
            if (src->shape[i] == target->shape[i]) continue;
            if (target->shape[i] != 1) return ZENU_ERR_SHAPE;
            axes[na] = i; keep[na] = 1; na++;
        }
    } else {
        // trailing dims must match exactly (is_include), leading axes are summed away
        for (int i = 0; i < target->ndim; i++)
            if (src->shape[diff + i] != target->shape[i]) return ZENU_ERR_SHAPE;
        for (int i = 0; i < diff; i++) { axes[na] = 0; keep[na] = 0; na++; }
    }

    zenu_tensor_t cur = *src;
    void *cur_buf = nullptr;  // workspace owning `cur`, if any
    for (int a = 0; a < na; a++) {
        int64_t oshape[kMaxDim];
        int ond = 0;
        for (int i = 0; i < cur.ndim; i++) {
            if (i == axes[a]) { if (keep[a]) oshape[ond++] = 1; continue; }
            oshape[ond++] = cur.shape[i];
        }
        const bool last = (a == na - 1);
        zenu_tensor_t dst;
        void *dst_buf = nullptr;
        if (last) {
            dst = *target;
        } else {
            int64_t cnt = 1;
            for (int i = 0; i < ond; i++) cnt *= oshape[i];
            rc = zenu_hip_malloc(&dst_buf, (size_t)(cnt ? cnt : 1) * esz, stream);
            if (rc) { if (cur_buf) zenu_hip_free(cur_buf, stream); return rc; }
            dst = default_view(dst_buf, ond, oshape);
        }
        rc = reduce_axis(kSum, dtype, &dst, nullptr, &cur, axes[a], s);
        if (cur_buf) zenu_hip_free(cur_buf, stream);
        cur_buf = dst_buf;
        if (rc) { if (cur_buf) zenu_hip_free(cur_buf, stream); return rc; }
        cur = dst;
    }
    return ZENU_OK;
}

}  // extern "C"
