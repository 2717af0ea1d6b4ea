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

template <typename T, int N> __device__ __forceinline__ Pack<T, N> splat(T s)
{
    Pack<T, N> r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = s;
    return r;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

}  // namespace zenu
