// vecmem.hpp -- 128-bit global memory accesses with an optional streaming (non-temporal) hint.
//
// Kernels that pass over operands once gain about 14 % of HBM bandwidth on MI355X when their
// loads and stores carry the `nt` hint (measured: 3-stream f32 add, 2^24 elements, 5.6 -> 6.4
// TB/s): the lines do not linger in L2 / the memory-side cache on their way through.  The hint
// is used only when an op moves more than kStreamBytes; smaller operands keep normal caching so
// that a following op can find them in L2.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace zenu {

constexpr int64_t kStreamBytes = 32ll << 20;  // about the aggregate L2 of the 8 XCDs

template <typename T, int N> struct NativeVec;
template <> struct NativeVec<float, 4> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct NativeVec<double, 2> { typedef double type __attribute__((ext_vector_type(2))); };
template <> struct NativeVec<float, 1> { typedef float type; };
template <> struct NativeVec<double, 1> { typedef double type; };

template <typename T> struct VecOf;
template <> struct VecOf<float> { static constexpr int N = 4; };
template <> struct VecOf<double> { static constexpr int N = 2; };

template <typename T, int N> struct Pack { T v[N]; };

template <typename T, int N, bool NT> __device__ __forceinline__ Pack<T, N> load_pack(const T *p)
{
    typedef typename NativeVec<T, N>::type V;
    V x;
    if constexpr (NT) x = __builtin_nontemporal_load(reinterpret_cast<const V *>(p));
    else x = *reinterpret_cast<const V *>(p);
    Pack<T, N> r;
    __builtin_memcpy(&r, &x, sizeof(V));
    return r;
}

template <typename T, int N, bool NT> __device__ __forceinline__ void store_pack(T *p, const Pack<T, N> &r)
{
    typedef typename NativeVec<T, N>::type V;
    V x;
    __builtin_memcpy(&x, &r, sizeof(V));
    if constexpr (NT) __builtin_nontemporal_store(x, reinterpret_cast<V *>(p));
    else *reinterpret_cast<V *>(p) = x;
}

// A 128-bit streaming store that is also written through (`sc1 nt`): for kernels with one load
// stream and one store stream.  Measured on a 2^24-element f32 copy, 64 threads x 1 vector, all 64
// combinations of {sc0, sc1, nt} on the loads and on the stores: only `nt` matters on the loads;
// on the stores `nt` gives 21.70 us, `sc1 nt` 21.22 us, `sc1` 21.3 us, none 22.8 us.  With two
// or more load streams beside the store (add: 31.8 us with `nt`, 32.1 - 32.2 us with `sc1 nt`;
// the seven streams of Adam: 114.5 against 115.8 us) plain `nt` stays ahead.  The compiler has no
// spelling for this combination, so the instruction is written out; the s_nop keeps the data
// registers untouched for the one wait state a 128-bit store needs after issue.
template <typename T, int N> __device__ __forceinline__ void store_pack_wt(T *p, const Pack<T, N> &r)
{
    static_assert(sizeof(T) * N == 16, "128-bit packs only");
    typedef typename NativeVec<T, N>::type V;
    V x;
    __builtin_memcpy(&x, &r, sizeof(V));
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 0" ::"v"(reinterpret_cast<V *>(p)), "v"(x) : "memory");
}

template <typename T, int N> __device__ __forceinline__ Pack<T, N> splat(T s)
{
    Pack<T, N> r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = s;
    return r;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace zenu
