// elementwise.hpp -- N-d elementwise engine for gfx950 (binary, scalar, unary, relu, clip, copy,
// broadcast).
//
// One Matrix-level call of the reference (add_array, mul_scalar, exp_array, relu, copy_from ...,
// zenu-matrix/src/operation/basic_operations.rs:278-381,512-611, relu.rs:169-242,
// copy_from.rs:211-267) becomes ONE launch here instead of one 1-D launch per row
// (zenu-matrix/src/with_clousers.rs:180-223).  After the host has folded the operands into a
// common iteration space (shape.cpp) one of four kernels runs:
//
//   contig : every operand is one contiguous run.  128-bit loads/stores; 64 threads x one vector
//            when one input streams (the shape that moves load + store traffic fastest), 256
//            threads x two vectors for two inputs and for tanh / sigmoid.           [HBM bound]
//   rows   : the innermost dim is contiguous (stride 1) or broadcast (stride 0) in every operand;
//            outer dims are arbitrary.  Covers row / column broadcast and row-sliced views.  The
//            outer index is decomposed once per thread, the inner dim is walked with 128-bit
//            accesses; a broadcast row stays in L2.                                   [HBM bound]
//   tile   : some input is contiguous along a different dim than the output (a transposed
//            operand).  64x64 tiles walked along diagonals, one thread per vector: the transposed
//            input is read along ITS contiguous dim with 128-bit loads in 128-byte segments,
//            turned through LDS (pitch 65 words, eight lanes per segment: no bank conflicts in
//            either direction, checked with the hardware counter), and every HBM access stays
//            coalesced.                                                               [HBM bound]
//   strided: anything else (a strided destination, gathers, views without a unit-stride dim):
//            lanes along the innermost dim whatever its stride, the outer index decomposed once
//            per thread, four elements per thread with the loads issued first.
//
// Arithmetic is plain IEEE with contraction off; + - * / sqrt are correctly rounded on gfx950,
// so results are bit-identical to the CPU loops of basic_operations.rs:93-181.
// This header holds the functors, the kernels and the launch logic; the entry points are spread over
// ew_binary.hip, ew_unary.hip, ew_unary_trig.hip and ew_misc.hip so that their template
// instantiations compile in parallel.
#pragma once
#include <math.h>

#include "common.hpp"
#include "vecmem.hpp"
#include "zmath.hpp"

#include <type_traits>

namespace zenu {
namespace {

constexpr int kBlock = 256;
#ifndef ZENU_EW_UNROLL
#define ZENU_EW_UNROLL 2
#endif
constexpr int kUnroll = ZENU_EW_UNROLL;
#ifndef ZENU_EW1_BLOCK
#define ZENU_EW1_BLOCK 64
#endif
#ifndef ZENU_EW1_UNROLL
#define ZENU_EW1_UNROLL 1
#endif

// ---- functors -----------------------------------------------------------------------------------

template <typename T, int OP> __device__ __forceinline__ T bin_apply(T a, T b)
{
    if constexpr (OP == ZENU_ADD) return a + b;
    else if constexpr (OP == ZENU_SUB) return a - b;
    else if constexpr (OP == ZENU_MUL) return a * b;
    else return a / b;
}

template <typename T, int OP> struct BinF {
    static constexpr int NIN = 2;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ T operator()(T a, T b) const { return bin_apply<T, OP>(a, b); }
};

// a op s; the scalar comes by value or from device memory (0-d tensor operand)
template <typename T, int OP> struct ScalarF {
    static constexpr int NIN = 1;
    T s;
    const T *sp;
    __device__ __forceinline__ void init() { if (sp) s = *sp; }
    __device__ __forceinline__ T operator()(T a, T) const { return bin_apply<T, OP>(a, s); }
};

__device__ __forceinline__ float dev_tanh(float x, const zmath::TanhRegs &rg) { return zmath::tanhf_simd(x, rg); }
__device__ __forceinline__ double dev_tanh(double x, const zmath::TanhRegs &) { return zmath::tanh_simd(x); }
__device__ __forceinline__ float dev_asin(float x) { return zmath::asinf_fdlibm(x); }
__device__ __forceinline__ double dev_asin(double x) { return asin(x); }
__device__ __forceinline__ float dev_acos(float x) { return zmath::acosf_fdlibm(x); }
__device__ __forceinline__ double dev_acos(double x) { return acos(x); }
__device__ __forceinline__ float dev_atan(float x) { return zmath::atanf_fdlibm(x); }
__device__ __forceinline__ double dev_atan(double x) { return atan(x); }
__device__ __forceinline__ float dev_sigmoid(float x, const zmath::TanhRegs &rg) { return zmath::sigmoidf_zenu(x, rg); }
__device__ __forceinline__ double dev_sigmoid(double x, const zmath::TanhRegs &) { return zmath::sigmoid_zenu(x); }

// what single functions carry besides: the f64 constants of the sine / cosine / tangent (in the functor, a
// kernel argument), the tables of the f64 sine / cosine and of the f32 arc tangent (in LDS); every other function nothing
template <typename T, int FN> struct UnaryExtra {
    __device__ __forceinline__ void init() {}
};
template <> struct UnaryExtra<float, ZENU_SIN> {
    zmath::SinCosCoef k;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ float sin(float x) const { return zmath::sinf_glibc(x, k); }
};
template <> struct UnaryExtra<float, ZENU_COS> {
    zmath::SinCosCoef k;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ float cos(float x) const { return zmath::cosf_glibc(x, k); }
};
template <> struct UnaryExtra<double, ZENU_SIN> {
    zmath::SinCos64Coef k;
    zmath::SinCos64Lds t;
    __device__ __forceinline__ void init() { t.init(); }
    __device__ __forceinline__ double sin(double x) const { return zmath::sin_glibc(x, t.tab, k); }
};
template <> struct UnaryExtra<double, ZENU_COS> {
    zmath::SinCos64Coef k;
    zmath::SinCos64Lds t;
    __device__ __forceinline__ void init() { t.init(); }
    __device__ __forceinline__ double cos(double x) const { return zmath::cos_glibc(x, t.tab, k); }
};
template <> struct UnaryExtra<float, ZENU_TAN> {
    zmath::TanfCoef tk;
    __device__ __forceinline__ void init() {}
};
template <> struct UnaryExtra<float, ZENU_ATAN> {
    zmath::AtanfLds t;
    __device__ __forceinline__ void init() { t.init(); }
};

template <typename T, int FN> struct UnaryF {
    static constexpr int NIN = 1;
    zmath::ExpLog<T> m;     // exp / log state (f32: tables in LDS)
    zmath::TanhRegs tr;     // f32 tanh / sigmoid / sinh / cosh: two constants held in vector registers
    UnaryExtra<T, FN> sc;   // f32 sin / cos / tan: the f64 constants, as data; f32 atan: its table
    __device__ __forceinline__ void init()
    {
        if constexpr (FN == ZENU_EXP || FN == ZENU_LOG || FN == ZENU_SINH || FN == ZENU_COSH)
            m.init(FN != ZENU_LOG, FN == ZENU_LOG);
        if constexpr (FN == ZENU_TANH || FN == ZENU_SIGMOID || FN == ZENU_SINH || FN == ZENU_COSH) tr.pin();
        sc.init();
    }
    __device__ __forceinline__ T operator()(T a, T) const
    {
        if constexpr (FN == ZENU_EXP) return m.exp(a);
        else if constexpr (FN == ZENU_LOG) return m.log(a);
        else if constexpr (FN == ZENU_TANH) return m.tanh(a, tr);
        else if constexpr (FN == ZENU_SQRT) return sqrt(a);
        else if constexpr (FN == ZENU_ABS) return fabs(a);
        else if constexpr (FN == ZENU_SIN) return sc.sin(a);
        else if constexpr (FN == ZENU_COS) return sc.cos(a);
        else if constexpr (FN == ZENU_TAN) {
            if constexpr (sizeof(T) == 4) return zmath::tanf_glibc(a, sc.tk);
            else return tan(a);
        }
        else if constexpr (FN == ZENU_ASIN) return dev_asin(a);
        else if constexpr (FN == ZENU_ACOS) return dev_acos(a);
        else if constexpr (FN == ZENU_ATAN) {
            if constexpr (sizeof(T) == 4) return zmath::atanf_fdlibm(a, sc.t.tab);
            else return dev_atan(a);
        }
        else if constexpr (FN == ZENU_SINH) return m.sinh(a, tr);
        else if constexpr (FN == ZENU_COSH) return m.cosh(a, tr);
        else return m.sigmoid(a, tr);
    }
};

// f32 tanh within 2 units in the last place of the host library's, evaluated in f64 (no
// counterpart in the reference; f64 goes to the exact tanh instead)
struct TanhUlp2F {
    static constexpr int NIN = 1;
    zmath::TanhUlp2Coef q;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ float operator()(float a, float) const { return zmath::tanhf_ulp2(a, q); }
};

template <typename T> struct PowF {
    static constexpr int NIN = 1;
    T s;
    zmath::Pow<T> m;        // f32: tables in LDS
    __device__ __forceinline__ void init() { m.init(); }
    __device__ __forceinline__ T operator()(T a, T) const { return m.pow(a, s); }
};

// relu.rs:44-48: the non-positive branch returns the PRODUCT alpha*x (-0.0 for alpha = 0)
template <typename T> struct ReluF {
    static constexpr int NIN = 1;
    T alpha;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ T operator()(T a, T) const { return (a > (T)0) ? a : alpha * a; }
};
// relu.rs:74-78
template <typename T> struct ReluMaskF {
    static constexpr int NIN = 1;
    T alpha;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ T operator()(T a, T) const { return (a > (T)0) ? (T)1 : alpha * (T)-1; }
};
// relu.rs backward: gx = gy * mask(x), the mask of ReluMaskF (zenu-autograd/src/activation/relu.rs:35-44)
template <typename T> struct ReluBwdF {
    static constexpr int NIN = 2;
    T alpha;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ T operator()(T gy, T x) const { return gy * ((x > (T)0) ? (T)1 : alpha * (T)-1); }
};
// backward of tanh (zenu-autograd/src/functions/tanh.rs:30-37): cosh(x), its square, gy / square --
// three ops there, each rounded once; the same roundings here in one pass
template <typename T> struct TanhBwdF {
    static constexpr int NIN = 2;
    zmath::ExpLog<T> m;
    __device__ __forceinline__ void init() { m.init(true, false); }
    __device__ __forceinline__ T operator()(T gy, T x) const
    {
        const T c = m.cosh(x);
        const T c2 = c * c;
        return gy / c2;
    }
};
// backward of the sigmoid composite (zenu-autograd/src/activation/sigmoid.rs:7-15) through its add,
// mul, tanh and mul nodes (functions/mul.rs:35-44): ((0.5 gy) / cosh(0.5 x)^2) 0.5, every step rounded
template <typename T> struct SigmoidBwdF {
    static constexpr int NIN = 2;
    zmath::ExpLog<T> m;
    __device__ __forceinline__ void init() { m.init(true, false); }
    __device__ __forceinline__ T operator()(T gy, T x) const
    {
        const T half = (T)0.5;
        const T xh = x * half;
        const T c = m.cosh(xh);
        const T c2 = c * c;
        const T g1 = half * gy;
        const T g2 = g1 / c2;
        return g2 * half;
    }
};
// clip.rs:50-57: below min -> min, above max -> max, NaN passes through
template <typename T> struct ClipF {
    static constexpr int NIN = 1;
    T lo, hi;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ T operator()(T a, T) const { return a < lo ? lo : (a > hi ? hi : a); }
};
// clip.rs:90-96: 0 outside [min, max], 1 inside (and for NaN)
template <typename T> struct ClipMaskF {
    static constexpr int NIN = 1;
    T lo, hi;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ T operator()(T a, T) const { return (a < lo || a > hi) ? (T)0 : (T)1; }
};
template <typename T> struct CopyF {
    static constexpr int NIN = 1;
    __device__ __forceinline__ void init() {}
    __device__ __forceinline__ T operator()(T a, T) const { return a; }
};

template <typename T, int N, typename F>
__device__ __forceinline__ Pack<T, N> apply_pack(const F &f, const Pack<T, N> &a, const Pack<T, N> &b)
{
    Pack<T, N> r;
#pragma unroll
    for (int i = 0; i < N; i++) r.v[i] = f(a.v[i], b.v[i]);
    return r;
}

// ---- kernel 1: contiguous ------------------------------------------------------------------------

// Workgroup shape per stream count (measured on 2^24 f32): two-stream ops (one load, one store)
// run best as many small workgroups with one vector per lane (copy: 6.26 TB/s at 64 x 1 against
// 5.92 at 256 x 2); three-stream ops are flat across shapes and keep 256 x 2.
// The VALU-bound functors (tanh, sigmoid) prefer the larger shape too.
template <typename F> struct IsValuBound { static constexpr bool value = false; };
template <typename T> struct IsValuBound<UnaryF<T, ZENU_TANH>> { static constexpr bool value = true; };
template <typename T> struct IsValuBound<UnaryF<T, ZENU_SIGMOID>> { static constexpr bool value = true; };
template <> struct IsValuBound<TanhUlp2F> { static constexpr bool value = true; };   // 24.4 us against 27.1 at 64 x 1
// f64 sine / cosine: a 3.5 KiB table per workgroup, and 60 f64 operations per element
template <> struct IsValuBound<UnaryF<double, ZENU_SIN>> { static constexpr bool value = true; };
template <> struct IsValuBound<UnaryF<double, ZENU_COS>> { static constexpr bool value = true; };
// measured on 2^24 elements (us at 64 x 1 -> at 256 x 2): f32 sin 25.6 -> 23.8, cos 25.9 -> 23.8, asin 25.4 -> 24.0,
// sinh 25.7 -> 25.2, cosh 26.4 -> 25.0; f64 sinh 63.9 -> 61.6, cosh 62.4 -> 55.4, sin 88.4 -> 49.8, cos 86.4 -> 49.6.
// (f32 acos 25.0 -> 26.3 and atan 23.5 -> 24.7 prefer the small shape, tan does not care.)
template <typename T> struct IsValuBound<UnaryF<T, ZENU_SINH>> { static constexpr bool value = true; };
template <typename T> struct IsValuBound<UnaryF<T, ZENU_COSH>> { static constexpr bool value = true; };
template <> struct IsValuBound<UnaryF<float, ZENU_SIN>> { static constexpr bool value = true; };
template <> struct IsValuBound<UnaryF<float, ZENU_COS>> { static constexpr bool value = true; };
template <> struct IsValuBound<UnaryF<float, ZENU_ASIN>> { static constexpr bool value = true; };
// f64 powf: 5 KiB of tables per workgroup (89 us at 64 x 1)
template <> struct IsValuBound<PowF<double>> { static constexpr bool value = true; };
template <typename T> struct IsValuBound<TanhBwdF<T>> { static constexpr bool value = true; };
template <typename T> struct IsValuBound<SigmoidBwdF<T>> { static constexpr bool value = true; };

template <typename F> struct ContigShape {
    static constexpr bool kSmall = F::NIN == 1 && !IsValuBound<F>::value;
    static constexpr int kBlock = kSmall ? ZENU_EW1_BLOCK : 256;
    static constexpr int kUnroll = kSmall ? ZENU_EW1_UNROLL : zenu::kUnroll;
};

template <typename T, int VEC, bool NT, typename F>
__global__ __launch_bounds__(ContigShape<F>::kBlock) void ew_contig_kernel(T *out, const T *a, const T *b,
                                                                         int64_t n, F f)
{
    constexpr int kBlock = ContigShape<F>::kBlock;
    constexpr int kUnroll = ContigShape<F>::kUnroll;
    constexpr int64_t kTile = (int64_t)kBlock * VEC * kUnroll;
    const int64_t base = (int64_t)blockIdx.x * kTile;
    const int tid = threadIdx.x;
    if (base + kTile <= n) {
        Pack<T, VEC> va[kUnroll], vb[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            int64_t i = base + ((int64_t)u * kBlock + tid) * VEC;
            va[u] = load_pack<T, VEC, NT>(a + i);
            if constexpr (F::NIN == 2) vb[u] = load_pack<T, VEC, NT>(b + i);
            else vb[u] = va[u];
        }
        f.init();   // after the loads are issued: what it fetches (a device scalar, a table) overlaps them
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            int64_t i = base + ((int64_t)u * kBlock + tid) * VEC;
            const Pack<T, VEC> r = apply_pack<T, VEC, F>(f, va[u], vb[u]);
            // one streamed input, one streamed output: the written-through streaming store (vecmem.hpp)
            if constexpr (NT && ContigShape<F>::kSmall && VEC > 1) store_pack_wt<T, VEC>(out + i, r);
            else store_pack<T, VEC, NT>(out + i, r);
        }
    } else {
        f.init();
        for (int u = 0; u < kUnroll; u++) {
            int64_t i = base + ((int64_t)u * kBlock + tid) * VEC;
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                if (i + j < n) {
                    T x = a[i + j];
                    T y = (F::NIN == 2) ? b[i + j] : x;
                    out[i + j] = f(x, y);
                }
            }
        }
    }
}

// ---- kernel 1b: flat, one operand periodic ---------------------------------------------------------
// The output and one input are contiguous and of full size; the other input varies along ONE of the
// (collapsed) dims only, where it is contiguous: a bias [1,C,1,1] on [N,C,H,W], a row [1,n] on
// [m,n], a column [m,1] on [m,n].  Flat index i reads y[(i / inner) % mid].  Indices are 32-bit
// (checked at launch).  With a one-input functor there is no x: the output is f(y) spread over the
// other dims (broadcast of a row, a column, a bias).  MODE 0: inner == 1 and mid % VEC == 0, y is read as vectors; MODE 1:
// inner % VEC == 0, one y per vector; MODE 2: inner >= VEC, a vector spans at most two y.

template <typename T, int VEC, bool NT, typename F, bool Y_FIRST, int MODE, int kBlock, int kUnroll>
__global__ __launch_bounds__(kBlock) void ew_periodic_kernel(T *out, const T *x, const T *y, uint32_t n,
                                                             uint32_t inner, uint32_t mid, F f)
{
    f.init();
    const uint32_t base = blockIdx.x * (uint32_t)(kBlock * VEC * kUnroll);
    auto y_of = [&](uint32_t i0) {
        Pack<T, VEC> yv;
        if constexpr (MODE == 0) {
            yv = load_pack<T, VEC, false>(y + i0 % mid);
        } else if constexpr (MODE == 1) {
            yv = splat<T, VEC>(y[(i0 / inner) % mid]);
        } else {
            const uint32_t q0 = i0 / inner, rem = i0 - q0 * inner, c0 = q0 % mid;
            const uint32_t c1 = c0 + 1 == mid ? 0 : c0 + 1;
            const T y0 = y[c0], y1 = y[c1];
#pragma unroll
            for (int j = 0; j < VEC; j++) yv.v[j] = rem + j >= inner ? y1 : y0;
        }
        return yv;
    };
    if (base + (uint32_t)(kBlock * VEC * kUnroll) <= n && base + (uint32_t)(kBlock * VEC * kUnroll) > base) {
        Pack<T, VEC> xv[kUnroll], yv[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint32_t i0 = base + (uint32_t)(u * kBlock + threadIdx.x) * VEC;
            yv[u] = y_of(i0);
            if constexpr (F::NIN == 2) xv[u] = load_pack<T, VEC, NT>(x + i0);
            else xv[u] = yv[u];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            const uint32_t i0 = base + (uint32_t)(u * kBlock + threadIdx.x) * VEC;
            const Pack<T, VEC> r = Y_FIRST ? apply_pack<T, VEC, F>(f, yv[u], xv[u]) : apply_pack<T, VEC, F>(f, xv[u], yv[u]);
            if constexpr (NT && VEC > 1) store_pack_wt<T, VEC>(out + i0, r);   // at most one streamed input beside the output
            else store_pack<T, VEC, NT>(out + i0, r);
        }
    } else {
        for (int u = 0; u < kUnroll; u++) {
            const uint64_t i0 = (uint64_t)base + (uint64_t)(u * kBlock + threadIdx.x) * VEC;
            for (int j = 0; j < VEC; j++) {
                const uint64_t i = i0 + j;
                if (i < n) {
                    const T ys = y[((uint32_t)i / inner) % mid];
                    const T xs = (F::NIN == 2) ? x[i] : ys;
                    out[i] = Y_FIRST ? f(ys, xs) : f(xs, ys);
                }
            }
        }
    }
}

// ---- shared index descriptor ---------------------------------------------------------------------

struct OuterDesc {
    int nouter;                          // number of outer dims (0..5)
    int64_t shape[kMaxDim];              // outer dims, slowest first
    int64_t stride[kMaxOperands][kMaxDim];
};

__device__ __forceinline__ void decompose(const OuterDesc &d, int64_t lin, int64_t &o0, int64_t &o1,
                                          int64_t &o2)
{
    o0 = o1 = o2 = 0;
    for (int k = d.nouter - 1; k >= 0; k--) {
        int64_t q, r;
        if (k == 0) {                 // the slowest dim takes what is left: no division
            q = 0;
            r = lin;
        } else if (lin < 0x7fffffffLL && d.shape[k] < 0x7fffffffLL) {
            uint32_t l32 = (uint32_t)lin, s32 = (uint32_t)d.shape[k];
            q = l32 / s32;
            r = l32 - (uint32_t)q * s32;
        } else {
            q = lin / d.shape[k];
            r = lin - q * d.shape[k];
        }
        o0 += r * d.stride[0][k];
        o1 += r * d.stride[1][k];
        o2 += r * d.stride[2][k];
        lin = q;
    }
}

// the same for an index that is known to fit 32 bits (then every dim does): no 64-bit division
__device__ __forceinline__ void decompose32(const OuterDesc &d, uint32_t lin, int64_t &o0, int64_t &o1,
                                            int64_t &o2)
{
    o0 = o1 = o2 = 0;
    for (int k = d.nouter - 1; k >= 0; k--) {
        uint32_t q = 0, r = lin;
        if (k != 0) {
            const uint32_t s32 = (uint32_t)d.shape[k];
            q = lin / s32;
            r = lin - q * s32;
        }
        o0 += (int64_t)r * d.stride[0][k];
        o1 += (int64_t)r * d.stride[1][k];
        o2 += (int64_t)r * d.stride[2][k];
        lin = q;
    }
}

// ---- kernel 2: rows (inner dim contiguous or broadcast) -------------------------------------------

struct RowsParams {
    OuterDesc outer;
    int64_t nrows;     // product of outer dims
    int64_t ncols;     // inner length
    int inner_a;       // inner stride of input a: 1 or 0
    int inner_b;       // inner stride of input b: 1 or 0
    int tx_shift;      // threads along the row = 1 << tx_shift (<= 256)
    int64_t col_tiles; // column tiles per row
    int grid2d;        // the grid is (column tiles, row blocks); else linear, column tiles fastest
};

// NTA / NTB: input a / b is streamed once (not broadcast along an outer dim); the output is
// streamed when either is.  Template parameters, because a run-time choice between a hinted and
// a plain load is merged by the compiler into one plain load.
template <typename T, int VEC, bool NTA, bool NTB, typename F, int kBlock, int kUnroll>
__global__ __launch_bounds__(kBlock) void ew_rows_kernel(T *out, const T *a, const T *b,
                                                         RowsParams p, F f)
{
    f.init();
    // The workgroups are short-lived, so the scalar work before the first load counts: every field
    // of the argument block that the common case needs is read here, together (one wait instead of
    // one per branch), and a 2-d grid spares the division of the workgroup index.
    int tx_shift = p.tx_shift, inner_a = p.inner_a, inner_b = p.inner_b, nouter = p.outer.nouter, grid2d = p.grid2d;
    int64_t nrows = p.nrows, ncols = p.ncols;
    int64_t so0 = p.outer.stride[0][0], sa0 = p.outer.stride[1][0], sb0 = p.outer.stride[2][0];
    asm volatile("" : : "s"(tx_shift), "s"(inner_a), "s"(inner_b), "s"(nouter), "s"(grid2d), "s"(nrows),
                      "s"(ncols), "s"(so0), "s"(sa0), "s"(sb0), "s"(out), "s"(a), "s"(b));
    const int tx_n = 1 << tx_shift;
    const int ty_n = kBlock >> tx_shift;
    const int tx = threadIdx.x & (tx_n - 1);
    const int ty = threadIdx.x >> tx_shift;
    uint32_t row_blk32, col_tile32;
    if (grid2d) {
        col_tile32 = blockIdx.x;
        row_blk32 = blockIdx.y;
    } else {
        // grid and col_tiles fit 32 bits (checked at launch)
        row_blk32 = blockIdx.x / (uint32_t)p.col_tiles;
        col_tile32 = blockIdx.x - row_blk32 * (uint32_t)p.col_tiles;
    }
    const int64_t col_tile = col_tile32;
    const int64_t row = (int64_t)row_blk32 * ty_n + ty;
    if (row >= nrows) return;
    int64_t oo, oa, ob;
    if (nouter == 1) {            // one outer dim: the row index is its coordinate
        oo = row * so0;
        oa = row * sa0;
        ob = row * sb0;
    } else {
        decompose(p.outer, row, oo, oa, ob);
    }
    T *orow = out + oo;
    const T *arow = a + oa;
    const T *brow = (F::NIN == 2) ? b + ob : arow;

    const int64_t cols_per_tile = (int64_t)tx_n * VEC * kUnroll;
    const int64_t c0 = col_tile * cols_per_tile;
    Pack<T, VEC> sa, sb;
    if (inner_a == 0) sa = splat<T, VEC>(arow[0]);
    if (F::NIN == 2 && inner_b == 0) sb = splat<T, VEC>(brow[0]);

    if (c0 + cols_per_tile <= ncols) {
        Pack<T, VEC> va[kUnroll], vb[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            int64_t c = c0 + ((int64_t)u * tx_n + tx) * VEC;
            va[u] = inner_a ? load_pack<T, VEC, NTA>(arow + c) : sa;
            if constexpr (F::NIN == 2) vb[u] = inner_b ? load_pack<T, VEC, NTB>(brow + c) : sb;
            else vb[u] = va[u];
        }
#pragma unroll
        for (int u = 0; u < kUnroll; u++) {
            int64_t c = c0 + ((int64_t)u * tx_n + tx) * VEC;
            const Pack<T, VEC> r = apply_pack<T, VEC, F>(f, va[u], vb[u]);
            if constexpr ((NTA != NTB || (F::NIN == 1 && NTA)) && VEC > 1) store_pack_wt<T, VEC>(orow + c, r);   // one streamed input
            else store_pack<T, VEC, (NTA || NTB)>(orow + c, r);
        }
    } else {
        for (int u = 0; u < kUnroll; u++) {
            int64_t c = c0 + ((int64_t)u * tx_n + tx) * VEC;
            if (c + VEC <= ncols) {
                Pack<T, VEC> x = inner_a ? load_pack<T, VEC, false>(arow + c) : sa;
                Pack<T, VEC> y = x;
                if constexpr (F::NIN == 2) y = inner_b ? load_pack<T, VEC, false>(brow + c) : sb;
                store_pack<T, VEC, false>(orow + c, apply_pack<T, VEC, F>(f, x, y));
            } else {
                for (int j = 0; j < VEC; j++) {
                    if (c + j < ncols) {
                        T x = inner_a ? arow[c + j] : sa.v[0];
                        T y = x;
                        if constexpr (F::NIN == 2) y = inner_b ? brow[c + j] : sb.v[0];
                        orow[c + j] = f(x, y);
                    }
                }
            }
        }
    }
}

// ---- kernel 3: 64x64 tiles with an LDS turn for transposed inputs ----------------------------------

// 64x64 tiles for f32 (16.6 KB of LDS per staged input), 32x32 for f64 (8.4 KB).  With one input
// (a transposed or permuted copy, a unary op on such a view) one thread per 16-byte vector of the
// tile (1024 / 512 threads): ONE vector per thread is the shape that streams one load and one
// store stream fastest here, as for the contiguous kernels.  Transposed copy of [4096,4096] f32 in
// a stand-alone probe, tiles walked along diagonals: 23.9 us, against 25.2 us with 256 threads and
// four vectors each; 32x32 tiles with 256 threads copy as fast (24.1 us) but leave operands that
// are not transposed with 128-byte row pieces.
// SMALL halves the edge (32 / 16): few tiles of a small matrix leave most CUs idle and make each workgroup a
// long chain; with a quarter of the tile per workgroup a transposed copy of [256,512] f32 takes 2.8 us
// against 3.3 us, of [784,512] 3.4 against 3.6 (the MLP step of a 512-wide layer issues eleven of them).
template <typename T, bool SMALL = false> struct TileOf { static constexpr int N = (sizeof(T) == 4 ? 64 : 32) / (SMALL ? 2 : 1); };
// With two inputs (three streams, a + b^T) two vectors per thread and operand at 512 threads are the
// fastest (stand-alone probe: 36.2 us with four at 256 threads, 35.5 us with two at 512, 35.7 us with
// one at 1024).
template <typename T, typename F, bool SMALL = false> struct TileThreads {
    static constexpr int kVecs = TileOf<T, SMALL>::N * TileOf<T, SMALL>::N / VecOf<T>::N;   // vectors per tile and operand
    static constexpr int value = (F::NIN == 1 || kVecs < 512) ? kVecs : 512;
};

enum { kWalkRows = 0, kWalkCols = 1, kWalkDiagonal = 2 };

struct TileParams {
    OuterDesc outer;      // batch dims (everything except the two tile dims)
    int64_t nbatch;
    int64_t R, C;         // tile dims: R = dim where transposed inputs are contiguous, C = output inner dim
    int64_t ldr[kMaxOperands];  // stride along R per operand
    int64_t ldc[kMaxOperands];  // stride along C per operand (1 for out; 0/1 direct; ld for transposed)
    int trans_a, trans_b;       // input goes through LDS
    int vec_ok;                 // alignment allows 128-bit accesses on full tiles
    int grid3d;                 // the grid is (tiles_c, tiles_r, nbatch); else linear, tiles_c fastest
    int walk;                   // order of the tiles: kWalkRows, kWalkCols (3-d grids only) or kWalkDiagonal
    int64_t tiles_r, tiles_c;
    uint32_t tiles_r_magic;     // min(floor(2^32 / tiles_r), 2^32 - 1): x mod tiles_r from one high multiply and a fix-up
};

template <typename T, bool NT, typename F, bool SMALL = false>
__global__ __launch_bounds__((TileThreads<T, F, SMALL>::value)) void ew_tile_kernel(T *out, const T *a, const T *b,
                                                                                  TileParams p, F f)
{
    constexpr int VEC = VecOf<T>::N;
    constexpr int kTile = TileOf<T, SMALL>::N;
    constexpr int kBlock = TileThreads<T, F, SMALL>::value;   // shadows the engine-wide 256
    constexpr int kPitch = kTile + 1;
    // Eight lanes cover one 128-byte segment of a tile row; 32 segments per pass.  With eight (not
    // sixteen) lanes along the vector dim the 32 lanes that the LDS serves together -- eight
    // vector positions x four rows -- fall into 32 different banks in the scatter (one element of
    // each lane's vector per instruction, rows one pitch apart) and in the gather alike; sixteen
    // lanes per row alias pairwise (4 m and 4 (m + 8) share a bank) whatever the pitch.
    constexpr int VPS = 8;                  // vectors per segment
    constexpr int SEG = kTile / (VPS * VEC);// segments per tile row (2)
    static_assert(SEG >= 1 && (kTile * SEG * VPS) % kBlock == 0, "tile geometry");
    // One staging tile per TRANSPOSED input, sized at launch: with a static tile per input, `a + b^T`
    // held 33 KB of LDS per workgroup for the one tile it uses, and four workgroups fit a CU instead
    // of eight (on a [4096,4096] f32 view of pitch 4160: 37.6 us against 36.0 us).
    extern __shared__ __align__(16) unsigned char lds_raw[];
    T *const lds_a = reinterpret_cast<T *>(lds_raw);
    f.init();

    // The order in which the tiles are walked decides which addresses the workgroups that run
    // together touch.  Row by row (consecutive workgroups along the output's rows) they read pieces
    // of a transposed input that lie a tile's height times ITS pitch apart; column by column they
    // write pieces (and read those of the other inputs) that far apart by the output's pitch; along
    // diagonals consecutive workgroups differ in both tile coordinates.  A distance that is a
    // multiple of 4 KiB lands on few memory channels, so the host picks the walk by the pitches
    // (transposed copy of 4096 x 4096 f32, pitch of the output / of the input in elements, us row by
    // row / column by column / diagonally: 4096 / 4096: 26.3 / 27.6 / 24.0; 4096 / 4352: 24.1 / 28.5 /
    // 26.7; 4352 / 4096: 26.4 / 24.9 / 28.3; 4352 / 4352: 24.1 / 25.3 / 31.2; 5120 / 5120: 26.6 / 29.4 / 25.8).
    // The grid is (column tiles, row tiles, batch) when that fits the grid limits, so that no
    // workgroup starts with a chain of integer divisions (in 64 bits they were most of this kernel's
    // instructions); otherwise a linear grid below 2^31, decomposed in 32 bits.
    // Every wave of the workgroup runs this scalar prologue, and nothing is in flight before it ends:
    // the fields it needs are read from the argument block together (one wait, not one per branch),
    // and the diagonal's remainder comes from a multiplier that the host prepared, not from a division.
    int grid3d = p.grid3d, vec_ok = p.vec_ok, nouter = p.outer.nouter, walk = p.walk;
    uint32_t ntr = (uint32_t)p.tiles_r, magic = p.tiles_r_magic;
    int64_t R = p.R, C = p.C;
    int64_t ldr0 = p.ldr[0], ldr1 = p.ldr[1], ldr2 = p.ldr[2], ldc1 = p.ldc[1], ldc2 = p.ldc[2];
    int trans_a = p.trans_a, trans_b = p.trans_b;
    asm volatile("" : : "s"(grid3d), "s"(vec_ok), "s"(nouter), "s"(walk), "s"(ntr), "s"(magic), "s"(R), "s"(C),
                      "s"(ldr0), "s"(ldr1), "s"(ldr2), "s"(ldc1), "s"(ldc2), "s"(trans_a), "s"(trans_b),
                      "s"(out), "s"(a), "s"(b));
    T *const lds_b = lds_a + ((F::NIN == 2 && trans_a) ? kTile * kPitch : 0);
    uint32_t tc32, tr32, batch32;
    if (grid3d) {
        const bool by_cols = walk == kWalkCols;       // then the grid is (row tiles, column tiles, batch)
        tc32 = by_cols ? blockIdx.y : blockIdx.x;
        tr32 = by_cols ? blockIdx.x : blockIdx.y;
        batch32 = blockIdx.z;
    } else {
        const uint32_t ntc = (uint32_t)p.tiles_c;
        const uint32_t q = blockIdx.x / ntc;
        tc32 = blockIdx.x - q * ntc;
        batch32 = q / ntr;
        tr32 = q - batch32 * ntr;
    }
    if (walk == kWalkDiagonal) {
        // (tr + tc) mod tiles_r: the multiplier is floor(2^32 / tiles_r) (2^32 - 1 for one tile row),
        // which is less than 1 below 2^32 / tiles_r, so for every 32-bit argument the quotient is
        // exact or one too small (the sum is below 2^32: both grids are)
        const uint32_t x = tr32 + tc32;
        const uint32_t q = __umulhi(x, magic);
        const uint32_t r = x - q * ntr;
        tr32 = r >= ntr ? r - ntr : r;
    }
    const int64_t tc = tc32, tr = tr32;
    int64_t oo = 0, oa = 0, ob = 0;
    if (nouter > 0) decompose32(p.outer, batch32, oo, oa, ob);
    const int64_t r0 = tr * kTile, c0 = tc * kTile;
    const int64_t nr = (R - r0 < kTile) ? R - r0 : kTile;
    const int64_t nc = (C - c0 < kTile) ? C - c0 : kTile;
    const bool full = (nr == kTile) & (nc == kTile) & (vec_ok != 0);
    const int tid = threadIdx.x;

    T *obase = out + oo + r0 * ldr0 + c0;
    const T *abase = a + oa + r0 * ldr1 + c0 * ldc1;
    const T *bbase = (F::NIN == 2) ? b + ob + r0 * ldr2 + c0 * ldc2 : abase;

    if (full) {
        // All global loads of the tile are issued first -- the transposed inputs along R (their
        // contiguous dim), the others along C -- so both streams are in flight together; then the
        // transposed ones are turned through LDS.
        // vector e = k * kBlock + tid of the tile: eight consecutive ones form a segment, the segments
        // of one segment column follow each other along the other dim
        constexpr int K = kTile * SEG * VPS / kBlock;   // vectors per thread and operand (1 or 4)
        const int seg_v = (tid % VPS) * VEC;            // vector position inside the segment
        auto other_of = [&](int k) { return ((k * kBlock + tid) / VPS) % kTile; };                  // position along the other dim
        auto vec_of = [&](int k) { return seg_v + (((k * kBlock + tid) / VPS) / kTile) * VPS * VEC; };  // element position along the vector dim
        const bool ta = trans_a != 0;
        const bool tb = (F::NIN == 2) && trans_b != 0;
        // A transposed input is read along R with its pitch ldc between the vectors, any other along C
        // with its pitch ldr: the same expression with the pitch selected, so the loads of one thread
        // follow each other without a branch between them.  (With a branch per load the compiler put a
        // wait for all earlier loads in front of each one: `a + b^T` 38.9 us instead of 36 us.)
        const int64_t pitch_a = ta ? ldc1 : ldr1;
        const int64_t pitch_b = tb ? ldc2 : ldr2;
        Pack<T, VEC> xa[K], xb[K];
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int o = other_of(k);
            const int lane_v = vec_of(k);
            xa[k] = load_pack<T, VEC, NT>(abase + lane_v + (int64_t)o * pitch_a);
            if constexpr (F::NIN == 2) xb[k] = load_pack<T, VEC, NT>(bbase + lane_v + (int64_t)o * pitch_b);
        }
        if (ta) {
#pragma unroll
            for (int k = 0; k < K; k++) {
                const int c = other_of(k);               // the loaded vector holds rows lane_v.. of column c
                const int lane_v = vec_of(k);
#pragma unroll
                for (int j = 0; j < VEC; j++) lds_a[(lane_v + j) * kPitch + c] = xa[k].v[j];
            }
        }
        if constexpr (F::NIN == 2) {
            if (tb) {
#pragma unroll
                for (int k = 0; k < K; k++) {
                    const int c = other_of(k);
                    const int lane_v = vec_of(k);
#pragma unroll
                    for (int j = 0; j < VEC; j++) lds_b[(lane_v + j) * kPitch + c] = xb[k].v[j];
                }
            }
        }
        __syncthreads();                                 // at least one input is transposed
        if (ta) {
#pragma unroll
            for (int k = 0; k < K; k++) {
                const int r = other_of(k);
                const int lane_v = vec_of(k);
#pragma unroll
                for (int j = 0; j < VEC; j++) xa[k].v[j] = lds_a[r * kPitch + lane_v + j];
            }
        }
        if constexpr (F::NIN == 2) {
            if (tb) {
#pragma unroll
                for (int k = 0; k < K; k++) {
                    const int r = other_of(k);
                    const int lane_v = vec_of(k);
#pragma unroll
                    for (int j = 0; j < VEC; j++) xb[k].v[j] = lds_b[r * kPitch + lane_v + j];
                }
            }
        }
#pragma unroll
        for (int k = 0; k < K; k++) {
            const int r = other_of(k);
            const int lane_v = vec_of(k);
            Pack<T, VEC> y = xa[k];
            if constexpr (F::NIN == 2) y = xb[k];
            store_pack<T, VEC, NT>(obase + (int64_t)r * ldr0 + lane_v, apply_pack<T, VEC, F>(f, xa[k], y));
        }
    } else {
        // Edge tiles and unaligned operands: element by element with bounds checks.  All loads of a
        // phase are issued before the first use (an element outside the tile reads the tile's first
        // one again and is dropped): with the loads inside the bounds check the compiler waits for each
        // before it issues the next, and a small matrix made of edge tiles only (the [512,10] weights of a
        // classifier head) took four memory round trips per phase instead of one.
        constexpr int E = kTile * kTile / kBlock;
        const bool ta = trans_a != 0;
        const bool tb = (F::NIN == 2) && trans_b != 0;
        if (ta || tb) {
            T va[E], vb[E];
#pragma unroll
            for (int i = 0; i < E; i++) {
                const int e = tid + i * kBlock;
                const int r = e % kTile, c = e / kTile;
                const bool ok = (r < nr) & (c < nc);
                const int64_t off_r = ok ? r : 0, off_c = ok ? c : 0;
                if (ta) va[i] = abase[off_r + off_c * ldc1];
                if constexpr (F::NIN == 2) {
                    if (tb) vb[i] = bbase[off_r + off_c * ldc2];
                }
            }
#pragma unroll
            for (int i = 0; i < E; i++) {
                const int e = tid + i * kBlock;
                const int r = e % kTile, c = e / kTile;
                if ((r < nr) & (c < nc)) {
                    if (ta) lds_a[r * kPitch + c] = va[i];
                    if constexpr (F::NIN == 2) {
                        if (tb) lds_b[r * kPitch + c] = vb[i];
                    }
                }
            }
            __syncthreads();
        }
        T x[E], y[E];
#pragma unroll
        for (int i = 0; i < E; i++) {
            const int e = tid + i * kBlock;
            const int c = e % kTile, r = e / kTile;
            const bool ok = (r < nr) & (c < nc);
            const int64_t off_r = ok ? r : 0, off_c = ok ? c : 0;
            if (!ta) x[i] = abase[off_r * ldr1 + off_c * ldc1];
            if constexpr (F::NIN == 2) {
                if (!tb) y[i] = bbase[off_r * ldr2 + off_c * ldc2];
            }
        }
#pragma unroll
        for (int i = 0; i < E; i++) {
            const int e = tid + i * kBlock;
            const int c = e % kTile, r = e / kTile;
            if ((r < nr) & (c < nc)) {
                if (ta) x[i] = lds_a[r * kPitch + c];
                if constexpr (F::NIN == 2) {
                    if (tb) y[i] = lds_b[r * kPitch + c];
                } else {
                    y[i] = x[i];
                }
                obase[(int64_t)r * ldr0 + c] = f(x[i], y[i]);
            }
        }
    }
}

// ---- kernel 4: strided rows (anything else) ----------------------------------------------------------
// Operands whose innermost (collapsed) dim has any stride: a strided destination (out[:, ::2] = ...),
// gathers (a[:, ::2] + b), views without a unit-stride dim.  The threads of a workgroup form
// (ty rows) x (tx columns) with the columns along the innermost dim, so consecutive lanes touch
// addresses one inner stride apart (as coalesced as the view allows); the outer index is
// decomposed once per thread, not per element, and an element's offset is column * stride.

struct StridedRowsParams {
    OuterDesc outer;
    int64_t nrows, ncols;
    int64_t inner[kMaxOperands];   // stride along the innermost dim per operand (any value)
    int tx_shift;
    int64_t col_tiles;
    int grid2d;        // the grid is (column tiles, row blocks); else linear, column tiles fastest
};

template <typename T, typename F, int kUnroll, bool NT>
__global__ __launch_bounds__(kBlock) void ew_strided_rows_kernel(T *out, const T *a, const T *b,
                                                                 StridedRowsParams p, F f)
{
    f.init();
    // as in the rows kernel: the argument block is read once, at the top, and a 2-d grid spares the division
    int tx_shift = p.tx_shift, nouter = p.outer.nouter, grid2d = p.grid2d;
    int64_t nrows = p.nrows, ncols = p.ncols;
    int64_t so0 = p.outer.stride[0][0], sa0 = p.outer.stride[1][0], sb0 = p.outer.stride[2][0];
    int64_t so = p.inner[0], sa = p.inner[1], sb = p.inner[2];
    asm volatile("" : : "s"(tx_shift), "s"(nouter), "s"(grid2d), "s"(nrows), "s"(ncols), "s"(so0), "s"(sa0),
                      "s"(sb0), "s"(so), "s"(sa), "s"(sb), "s"(out), "s"(a), "s"(b));
    const int tx_n = 1 << tx_shift;
    const int ty_n = kBlock >> tx_shift;
    const int tx = threadIdx.x & (tx_n - 1);
    const int ty = threadIdx.x >> tx_shift;
    uint32_t row_blk32, col_tile32;
    if (grid2d) {
        col_tile32 = blockIdx.x;
        row_blk32 = blockIdx.y;
    } else {
        row_blk32 = blockIdx.x / (uint32_t)p.col_tiles;   // grid and col_tiles fit 32 bits (checked at launch)
        col_tile32 = blockIdx.x - row_blk32 * (uint32_t)p.col_tiles;
    }
    const int64_t col_tile = col_tile32;
    const int64_t row = (int64_t)row_blk32 * ty_n + ty;
    if (row >= nrows) return;
    int64_t oo, oa, ob;
    if (nouter == 1) {
        oo = row * so0;
        oa = row * sa0;
        ob = row * sb0;
    } else {
        decompose(p.outer, row, oo, oa, ob);
    }
    T *orow = out + oo;
    const T *arow = a + oa;
    const T *brow = (F::NIN == 2) ? b + ob : arow;
    const int64_t c0 = col_tile * ((int64_t)tx_n * kUnroll) + tx;
    T x[kUnroll], y[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {          // all loads of the thread first
        // A column past the end reads the last one again (and stores nothing): with the loads under
        // the bounds check the compiler waits for the first before it issues the others.
        const int64_t c = c0 + (int64_t)u * tx_n;
        const int64_t cl = c < ncols ? c : ncols - 1;
        x[u] = load_pack<T, 1, NT>(arow + cl * sa).v[0];
        if constexpr (F::NIN == 2) y[u] = load_pack<T, 1, NT>(brow + cl * sb).v[0];
        else y[u] = x[u];
    }
#pragma unroll
    for (int u = 0; u < kUnroll; u++) {
        const int64_t c = c0 + (int64_t)u * tx_n;
        if (c < ncols) {
            Pack<T, 1> r;
            r.v[0] = f(x[u], y[u]);
            store_pack<T, 1, NT>(orow + c * so, r);
        }
    }
}

// ---- host dispatch ---------------------------------------------------------------------------------

template <typename T, typename F> int launch_ew(EwProblem &p, F f, hipStream_t stream)
{
    constexpr int VEC = VecOf<T>::N;
    ew_collapse(p);
    if (p.numel == 0) return ZENU_OK;
    if (int rc = ew_check_alias(p, sizeof(T))) return rc;
    T *out = static_cast<T *>(p.ptr[0]);
    const T *a = static_cast<const T *>(p.ptr[1]);
    const T *b = (F::NIN == 2) ? static_cast<const T *>(p.ptr[2]) : a;
    const int nin = F::NIN;
    // operands are streamed once: hint the caches when the op is larger than they are
    const bool nt = p.numel * (int64_t)sizeof(T) * (nin + 1) >= kStreamBytes;
    if (p.ndim == 0) {  // a single element
        p.ndim = 1;
        p.shape[0] = 1;
        for (int o = 0; o < p.nops; o++) p.stride[o][0] = 1;
    }
    const int last = p.ndim - 1;

    // contig
    bool all_unit = p.ndim == 1;
    for (int o = 0; o <= nin && all_unit; o++)
        if (p.stride[o][0] != 1) all_unit = false;
    if (all_unit) {
        const int64_t n = p.numel;
        bool vec = aligned16(out) && aligned16(a) && aligned16(b);
        if (vec) {
            constexpr int cb = ContigShape<F>::kBlock, cu = ContigShape<F>::kUnroll;
            int64_t tile = (int64_t)cb * VEC * cu;
            int64_t grid = (n + tile - 1) / tile;
            if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
            if (nt) ew_contig_kernel<T, VEC, true, F><<<(unsigned)grid, cb, 0, stream>>>(out, a, b, n, f);
            else    ew_contig_kernel<T, VEC, false, F><<<(unsigned)grid, cb, 0, stream>>>(out, a, b, n, f);
        } else {
            constexpr int cb = ContigShape<F>::kBlock, cu = ContigShape<F>::kUnroll;
            int64_t tile = (int64_t)cb * cu;
            int64_t grid = (n + tile - 1) / tile;
            if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
            ew_contig_kernel<T, 1, false, F><<<(unsigned)grid, cb, 0, stream>>>(out, a, b, n, f);
        }
        ZENU_LAUNCH_CHECK();
        return ZENU_OK;
    }

    // flat with one periodic operand (bias over channels, a row or a column over a matrix)
    {
        if (p.numel < ((int64_t)1 << 32) - 65536 && aligned16(out)) {
            auto flat = [&](int o) {
                int64_t want = 1;
                for (int d = p.ndim - 1; d >= 0; d--) {
                    if (p.stride[o][d] != want) return false;
                    want *= p.shape[d];
                }
                return true;
            };
            auto period_dim = [&](int o) {   // the one dim along which operand o varies (stride 1), else -1
                int m = -1;
                for (int d = 0; d < p.ndim; d++) {
                    if (p.stride[o][d] == 0) continue;
                    if (p.stride[o][d] != 1 || m >= 0) return -1;
                    m = d;
                }
                return m;
            };
            int yo = 0, m = -1;
            if (nin == 1) {
                if (flat(0) && !flat(1) && (m = period_dim(1)) >= 0) yo = 1;
            } else if (flat(0) && flat(1) && (m = period_dim(2)) >= 0) yo = 2;
            else if (flat(0) && flat(2) && (m = period_dim(1)) >= 0) yo = 1;
            if (yo) {
                const T *x = yo == 2 ? a : b, *y = yo == 2 ? b : a;   // one input: x == y == a, x is not read
                int64_t inner = 1;
                for (int d = m + 1; d < p.ndim; d++) inner *= p.shape[d];
                const int64_t mid = p.shape[m];
                const int mode = (inner == 1 && mid % VEC == 0 && aligned16(y)) ? 0
                                 : (inner % VEC == 0)                           ? 1
                                 : (inner >= VEC)                               ? 2 : -1;
                if (mode >= 0 && aligned16(x)) {
                    // one load and one store stream: the small workgroup shape of the unary ops when y comes as
                    // vectors (22.4 against 23.5 us on [4096,4096] + [1,4096]); with the index divisions of
                    // the other modes the larger shape is the better one (16.4 against 17.0 us on a
                    // [64,256,28,28] bias add)
                    const uint32_t n32 = (uint32_t)p.numel, in32 = (uint32_t)inner, mid32 = (uint32_t)mid;
                    auto go = [&](auto yfirst_c, auto mode_c) {
                        constexpr bool YF = decltype(yfirst_c)::value;
                        constexpr int MODE = decltype(mode_c)::value;
                        // a lone store stream (one-input functor) keeps the larger shape, like the fill kernel
                        constexpr bool small = MODE == 0 && !IsValuBound<F>::value && F::NIN == 2;
                        constexpr int B = small ? ZENU_EW1_BLOCK : 256, U = small ? ZENU_EW1_UNROLL : 2;
                        const int64_t tile = (int64_t)B * VEC * U;
                        const unsigned grid = (unsigned)((p.numel + tile - 1) / tile);
                        if (nt) ew_periodic_kernel<T, VEC, true, F, YF, MODE, B, U><<<grid, B, 0, stream>>>(out, x, y, n32, in32, mid32, f);
                        else    ew_periodic_kernel<T, VEC, false, F, YF, MODE, B, U><<<grid, B, 0, stream>>>(out, x, y, n32, in32, mid32, f);
                    };
                    auto by_mode = [&](auto yfirst_c) {
                        if (mode == 0) go(yfirst_c, std::integral_constant<int, 0>());
                        else if (mode == 1) go(yfirst_c, std::integral_constant<int, 1>());
                        else go(yfirst_c, std::integral_constant<int, 2>());
                    };
                    if (yo == 1) by_mode(std::true_type());
                    else by_mode(std::false_type());
                    ZENU_LAUNCH_CHECK();
                    return ZENU_OK;
                }
            }
        }
    }

    const bool out_inner_unit = p.stride[0][last] == 1;
    bool inner_01 = out_inner_unit;
    for (int o = 1; o <= nin && inner_01; o++)
        if (p.stride[o][last] != 0 && p.stride[o][last] != 1) inner_01 = false;

    if (inner_01) {
        RowsParams rp;
        rp.outer.nouter = p.ndim - 1;
        for (int d = 0; d < kMaxDim; d++) {
            rp.outer.shape[d] = d < p.ndim - 1 ? p.shape[d] : 1;
            for (int o = 0; o < kMaxOperands; o++)
                rp.outer.stride[o][d] = (d < p.ndim - 1 && o < p.nops) ? p.stride[o][d] : 0;
        }
        rp.ncols = p.shape[last];
        rp.nrows = p.numel / rp.ncols;
        rp.inner_a = (int)p.stride[1][last];
        rp.inner_b = nin == 2 ? (int)p.stride[2][last] : 1;
        bool nta = nt && rp.inner_a == 1, ntb = nt && nin == 2 && rp.inner_b == 1;
        for (int d = 0; d < p.ndim - 1; d++) {
            if (p.stride[1][d] == 0) nta = false;   // re-read for every outer index: keep it cached
            if (nin == 2 && p.stride[2][d] == 0) ntb = false;
        }
        bool vec = aligned16(out) && (rp.ncols % VEC == 0);
        for (int o = 1; o <= nin && vec; o++)
            if (p.stride[o][last] == 1 && !aligned16(p.ptr[o])) vec = false;
        for (int d = 0; d < p.ndim - 1 && vec; d++) {
            if (p.stride[0][d] % VEC) vec = false;
            for (int o = 1; o <= nin; o++)
                if (p.stride[o][last] == 1 && p.stride[o][d] % VEC) vec = false;
        }
        const int v = vec ? VEC : 1;
        int64_t vcols = (rp.ncols + v - 1) / v;
        // full-size streams of this launch: the output plus every input that is neither a scalar
        // per row nor re-read for every outer index; exactly two of them (one load, one store per
        // element) take the small workgroup shape.  A lone store stream (broadcast of a row) does
        // not: measured 13.0 us at 256 threads x 2 vectors against 18.7 us at 64 x 1 for 64 MiB
        int streams = 1;
        for (int o = 1; o <= nin; o++) {
            bool full = p.stride[o][last] == 1;
            for (int d = 0; d < p.ndim - 1; d++)
                if (p.stride[o][d] == 0 && p.shape[d] > 1) full = false;
            if (full) streams++;
        }
        const bool small = streams == 2 && !IsValuBound<F>::value;
        auto launch = [&](auto block_c, auto unroll_c) -> int {
            constexpr int B = decltype(block_c)::value, U = decltype(unroll_c)::value;
            int shift = 0;
            while ((1 << shift) < B && ((int64_t)1 << shift) < vcols) shift++;
            rp.tx_shift = shift;
            int64_t cols_per_tile = ((int64_t)1 << shift) * v * U;
            rp.col_tiles = (rp.ncols + cols_per_tile - 1) / cols_per_tile;
            int64_t rows_per_blk = B >> shift;
            const int64_t row_blks = (rp.nrows + rows_per_blk - 1) / rows_per_blk;
            if (row_blks * rp.col_tiles > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
            rp.grid2d = row_blks <= 65535 ? 1 : 0;
            const dim3 grid = rp.grid2d ? dim3((unsigned)rp.col_tiles, (unsigned)row_blks) : dim3((unsigned)(row_blks * rp.col_tiles));
            if (!vec)            ew_rows_kernel<T, 1, false, false, F, B, U><<<grid, B, 0, stream>>>(out, a, b, rp, f);
            else if (nta && ntb) ew_rows_kernel<T, VEC, true, true, F, B, U><<<grid, B, 0, stream>>>(out, a, b, rp, f);
            else if (nta)        ew_rows_kernel<T, VEC, true, false, F, B, U><<<grid, B, 0, stream>>>(out, a, b, rp, f);
            else if (ntb)        ew_rows_kernel<T, VEC, false, true, F, B, U><<<grid, B, 0, stream>>>(out, a, b, rp, f);
            else                 ew_rows_kernel<T, VEC, false, false, F, B, U><<<grid, B, 0, stream>>>(out, a, b, rp, f);
            return ZENU_OK;
        };
        int rc = small ? launch(std::integral_constant<int, ZENU_EW1_BLOCK>(), std::integral_constant<int, ZENU_EW1_UNROLL>())
                       : launch(std::integral_constant<int, kBlock>(), std::integral_constant<int, kUnroll>());
        if (rc) return rc;
        ZENU_LAUNCH_CHECK();
        return ZENU_OK;
    }

    // tile: every input is either inner-{0,1} or unit-stride along one common other dim `ri`
    if (out_inner_unit && p.ndim >= 2) {
        int ri = -1;
        bool ok = true;
        int trans[kMaxOperands] = {0, 0, 0};
        for (int o = 1; o <= nin && ok; o++) {
            int64_t s = p.stride[o][last];
            if (s == 0 || s == 1) continue;
            int found = -1;
            for (int d = 0; d < last; d++)
                if (p.stride[o][d] == 1) { found = d; break; }
            if (found < 0 || (ri >= 0 && ri != found)) ok = false;
            else { ri = found; trans[o] = 1; }
        }
        if (ok && ri >= 0) {
            TileParams tp;
            int k = 0;
            for (int d = 0; d < kMaxDim; d++) {
                tp.outer.shape[d] = 1;
                for (int o = 0; o < kMaxOperands; o++) tp.outer.stride[o][d] = 0;
            }
            for (int d = 0; d < last; d++) {
                if (d == ri) continue;
                tp.outer.shape[k] = p.shape[d];
                for (int o = 0; o < p.nops; o++) tp.outer.stride[o][k] = p.stride[o][d];
                k++;
            }
            tp.outer.nouter = k;
            tp.R = p.shape[ri];
            tp.C = p.shape[last];
            tp.nbatch = p.numel / (tp.R * tp.C);
            for (int o = 0; o < kMaxOperands; o++) {
                tp.ldr[o] = o < p.nops ? p.stride[o][ri] : 0;
                tp.ldc[o] = o < p.nops ? p.stride[o][last] : 0;
            }
            tp.trans_a = trans[1];
            tp.trans_b = nin == 2 ? trans[2] : 0;
            bool vec = true;
            for (int o = 0; o <= nin && vec; o++) {
                if (!aligned16(p.ptr[o])) vec = false;
                // every stride that moves a vector's base address must keep 16 B alignment
                for (int d = 0; d < p.ndim && vec; d++) {
                    int64_t s = p.stride[o][d];
                    if (s == 1 || s == 0) continue;
                    if (s % VEC) vec = false;
                }
            }
            // the vector path reads whole vectors along C from the inputs that are not transposed: one
            // that is broadcast along C (a column beside a transposed operand) takes the element path
            for (int o = 1; o <= nin; o++)
                if (!trans[o] && tp.ldc[o] == 0) vec = false;
            tp.vec_ok = vec ? 1 : 0;
            // tile edge: halved when the full-size tiles would not give every CU two workgroups
            auto launch_tiles = [&](auto small_c) -> int {
                constexpr bool SMALL = decltype(small_c)::value;
                constexpr int kTile = TileOf<T, SMALL>::N;
                tp.tiles_r = (tp.R + kTile - 1) / kTile;
                tp.tiles_c = (tp.C + kTile - 1) / kTile;
                {
                    const uint64_t m = (1ull << 32) / (uint64_t)tp.tiles_r;
                    tp.tiles_r_magic = m > 0xffffffffull ? 0xffffffffu : (uint32_t)m;
                }
                int64_t grid = tp.nbatch * tp.tiles_r * tp.tiles_c;
                if (grid > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
                tp.grid3d = (tp.tiles_r <= 65535 && tp.nbatch <= 65535) ? 1 : 0;
                // Row by row unless a transposed input's pitch is within one row piece of a multiple of
                // 4 KiB; then column by column if no other operand's pitch is, else along diagonals.
                auto near_4k = [](int64_t elems) {
                    const int64_t r = ((elems < 0 ? -elems : elems) * (int64_t)sizeof(T)) % 4096;
                    return (r < 4096 - r ? r : 4096 - r) < kTile * (int64_t)sizeof(T);
                };
                bool trans_near = false, direct_near = near_4k(tp.ldr[0]);
                for (int o = 1; o <= nin; o++) {
                    if (trans[o]) trans_near = trans_near || near_4k(tp.ldc[o]);
                    else if (tp.ldc[o] == 1) direct_near = direct_near || near_4k(tp.ldr[o]);
                }
                tp.walk = !trans_near ? kWalkRows
                          : (!direct_near && tp.grid3d && tp.tiles_c <= 65535) ? kWalkCols : kWalkDiagonal;
                const bool by_cols = tp.walk == kWalkCols;
                const dim3 g = !tp.grid3d ? dim3((unsigned)grid)
                               : by_cols ? dim3((unsigned)tp.tiles_r, (unsigned)tp.tiles_c, (unsigned)tp.nbatch)
                                         : dim3((unsigned)tp.tiles_c, (unsigned)tp.tiles_r, (unsigned)tp.nbatch);
                const size_t lds = (size_t)(tp.trans_a + tp.trans_b) * kTile * (kTile + 1) * sizeof(T);
                constexpr int kThreads = TileThreads<T, F, SMALL>::value;
                if (nt) ew_tile_kernel<T, true, F, SMALL><<<g, kThreads, lds, stream>>>(out, a, b, tp, f);
                else    ew_tile_kernel<T, false, F, SMALL><<<g, kThreads, lds, stream>>>(out, a, b, tp, f);
                return ZENU_OK;
            };
            constexpr int kFullTile = TileOf<T>::N;
            const int64_t full_tiles = tp.nbatch * ((tp.R + kFullTile - 1) / kFullTile) * ((tp.C + kFullTile - 1) / kFullTile);
            const int rc_tiles = full_tiles < 2 * (int64_t)device_info().num_cus ? launch_tiles(std::true_type())
                                                                                  : launch_tiles(std::false_type());
            if (rc_tiles) return rc_tiles;
            ZENU_LAUNCH_CHECK();
            return ZENU_OK;
        }
    }

    // strided rows: rows = everything but the innermost dim
    StridedRowsParams sp;
    sp.outer.nouter = p.ndim - 1;
    for (int d = 0; d < kMaxDim; d++) {
        sp.outer.shape[d] = d < p.ndim - 1 ? p.shape[d] : 1;
        for (int o = 0; o < kMaxOperands; o++)
            sp.outer.stride[o][d] = (d < p.ndim - 1 && o < p.nops) ? p.stride[o][d] : 0;
    }
    sp.ncols = p.shape[last];
    sp.nrows = p.numel / sp.ncols;
    for (int o = 0; o < kMaxOperands; o++) sp.inner[o] = o < p.nops ? p.stride[o][last] : 0;
    constexpr int kStridedUnroll = 4;
    int shift = 0;
    while ((1 << shift) < kBlock && ((int64_t)1 << shift) < sp.ncols) shift++;
    sp.tx_shift = shift;
    const int64_t cols_per_tile = ((int64_t)1 << shift) * kStridedUnroll;
    sp.col_tiles = (sp.ncols + cols_per_tile - 1) / cols_per_tile;
    const int64_t rows_per_blk = kBlock >> shift;
    const int64_t row_blks = (sp.nrows + rows_per_blk - 1) / rows_per_blk;
    if (row_blks * sp.col_tiles > 0x7fffffffLL || sp.col_tiles > 0x7fffffffLL) return ZENU_ERR_UNSUPPORTED;
    sp.grid2d = row_blks <= 65535 ? 1 : 0;
    const dim3 grid = sp.grid2d ? dim3((unsigned)sp.col_tiles, (unsigned)row_blks) : dim3((unsigned)(row_blks * sp.col_tiles));
    // streaming hint only when every cache line an access touches is used up by the same wavefront
    // (small inner strides); with large strides the neighbours of an element belong to other rows
    bool snt = nt;
    for (int o = 0; o <= nin; o++)
        if (sp.inner[o] > 4) snt = false;
    if (snt) ew_strided_rows_kernel<T, F, kStridedUnroll, true><<<grid, kBlock, 0, stream>>>(out, a, b, sp, f);
    else     ew_strided_rows_kernel<T, F, kStridedUnroll, false><<<grid, kBlock, 0, stream>>>(out, a, b, sp, f);
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

// problem builders -----------------------------------------------------------------------------------

void init_problem(EwProblem &p, const zenu_tensor_t &to, int nops)
{
    p.nops = nops;
    p.ndim = to.ndim;
    for (int d = 0; d < to.ndim; d++) p.shape[d] = to.shape[d];
    for (int d = to.ndim; d < kMaxDim; d++) p.shape[d] = 1;
    for (int o = 0; o < kMaxOperands; o++) {
        p.ptr[o] = nullptr;
        for (int d = 0; d < kMaxDim; d++) p.stride[o][d] = 0;
    }
    ew_set_operand(p, 0, to, to.ndim, to.shape);
    // the output is never broadcast: keep its own strides even on size-1 dims
    for (int d = 0; d < to.ndim; d++) p.stride[0][d] = to.stride[d];
}

template <typename T, typename F>
int run1(const zenu_tensor_t &to, const zenu_tensor_t &in, F f, hipStream_t s)
{
    EwProblem p;
    init_problem(p, to, 2);
    ew_set_operand(p, 1, in, to.ndim, to.shape);
    return launch_ew<T, F>(p, f, s);
}

template <typename T, typename F>
int run2(const zenu_tensor_t &to, const zenu_tensor_t &x, const zenu_tensor_t &y, F f, hipStream_t s)
{
    EwProblem p;
    init_problem(p, to, 3);
    ew_set_operand(p, 1, x, to.ndim, to.shape);
    ew_set_operand(p, 2, y, to.ndim, to.shape);
    return launch_ew<T, F>(p, f, s);
}

int check2(const zenu_tensor_t *a, const zenu_tensor_t *b)
{
    int rc = validate_tensor(a);
    if (rc) return rc;
    return validate_tensor(b);
}

}  // namespace
}  // namespace zenu
