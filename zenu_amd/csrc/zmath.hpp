// zmath.hpp -- the transcendental functions of the kernels, bit-compatible with the host libm that
// the reference's CPU path calls (Rust f32::tanh / exp / ln / powf ... -> libm tanhf / expf / logf /
// powf ...; glibc 2.35 is what this image ships).
//
//   f32: tanh, expm1, exp, log, powf, sinh, cosh, sin, cos, tan, atan, asin, acos, the sigmoid composite
//   f64: tanh, expm1, exp, log, pow, sinh, cosh, sin, cos, the sigmoid composite
//   (f64 tan, asin, acos, atan are not here: the host's routines rest on tables and fitted coefficients
//   that their sources give only as literals; the kernels call the device math library for them)
//
// Why not the device math library: ZeNu's sigmoid is the composite 0.5 + 0.5*tanh(0.5*x)
// (zenu-autograd/src/activation/sigmoid.rs:7-15).  For negative x the final add cancels, so a
// 1-ulp difference in tanh becomes tens of ulps in the sigmoid; parity therefore needs the
// same tanh bits as the CPU path, not merely an accurate tanh.  The other functions follow the
// same idea: each restates the algorithm the host libm uses (fdlibm's float and double routines,
// ARM's table-driven expf / logf / powf / sinf / cosf / exp / log / pow and IBM's double sin / cos as
// glibc carries them; tables rebuilt from their definitions, see tablegen/), with the fused
// multiply-adds exactly where the x86-64 build that CPUs with FMA select has them, so host and
// device produce identical bits.
//
// tanh, the first of them: the classic fdlibm single-precision tanhf / expm1f (Sun Microsystems, 1993):
//   tanh(x) = sign(x) * { |x| < 2^-55 : |x|*(1+|x|)
//                         |x| <  1    : -t/(t+2),   t = expm1(-2|x|)
//                         |x| <  22   : 1 - 2/(t+2), t = expm1( 2|x|)
//                         else        : 1 }
//   expm1(x): x = k*ln2 + r, |r| <= 0.5 ln2; R1(r*r) rational correction; scale by 2^k.
// Everything there is plain IEEE f32 arithmetic (+,-,*,/ correctly rounded, no contraction).
//
// The host build of this header is compared with the host libm by tests/native/zmath_host_check.cpp
// (tests/test_host_native.py runs it on a sample; on every f32 bit pattern and on 2e10 sampled
// f64 inputs it was run during development, without a mismatch).
//
// The header can be instantiated a second time under another namespace (define ZMATH_NAMESPACE
// before including it again): selfcheck.hip does that with ZMATH_EXACT_DIVISION, which makes the
// short division and square root below the IEEE operations, to compare the two builds of every
// function on every f32 argument on the device.
#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(ZMATH_NAMESPACE)
#define ZMATH_NS ZMATH_NAMESPACE
#define ZMATH_EMIT 1
#elif !defined(ZMATH_HPP_INCLUDED)
#define ZMATH_HPP_INCLUDED
#define ZMATH_NS zmath
#define ZMATH_EMIT 1
#endif
#ifdef ZMATH_EMIT

#undef ZM_HD
#undef ZM_RARE
#if defined(__HIPCC__)
#define ZM_HD __host__ __device__ __forceinline__
// a rarely taken path kept out of line: one copy per kernel instead of one per element of the
// unrolled loop (the branchy fdlibm forms are thousands of instructions when inlined eight times)
#define ZM_RARE __host__ __device__ __attribute__((noinline)) static
#else
#define ZM_HD static inline
#define ZM_RARE static
#endif

namespace ZMATH_NS {

ZM_HD uint32_t f2u(float f)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __float_as_uint(f);
#else
    uint32_t u;
    memcpy(&u, &f, 4);
    return u;
#endif
}
ZM_HD float u2f(uint32_t u)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __uint_as_float(u);
#else
    float f;
    memcpy(&f, &u, 4);
    return f;
#endif
}

// expm1f for finite |x| < 88 (callers here pass |x| < 44); follows fdlibm s_expm1f.c.
ZM_HD float expm1f_fdlibm(float x)
{
    const float one = 1.0f, tiny = 1.0e-30f, huge = 1.0e+30f;
    const float o_threshold = u2f(0x42b17180u);   // 8.8721679688e+01
    const float ln2_hi = u2f(0x3f317180u);        // 6.9313812256e-01
    const float ln2_lo = u2f(0x3717f7d1u);        // 9.0580006145e-06
    const float invln2 = u2f(0x3fb8aa3bu);        // 1.4426950216e+00
    const float Q1 = u2f(0xbd088889u);            // -3.3333335072e-02
    const float Q2 = u2f(0x3ad00d01u);            //  1.5873016091e-03
    const float Q3 = u2f(0xb8a670cdu);            // -7.9365076090e-05
    const float Q4 = u2f(0x36867e54u);            //  4.0082177293e-06
    const float Q5 = u2f(0xb457edbbu);            // -2.0109921195e-07

    float y, hi, lo, c = 0.0f, t, e, hxs, hfx, r1;
    int32_t k;
    uint32_t hx = f2u(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;

    // huge and non-finite arguments
    if (hx >= 0x4195b844u) {            // |x| >= 27*ln2
        if (hx >= 0x42b17218u) {        // |x| >= 88.721...
            if (hx > 0x7f800000u) return x + x;                     // NaN
            if (hx == 0x7f800000u) return (xsb == 0) ? x : -1.0f;   // +-inf
            if (x > o_threshold) return huge * huge;                // overflow
        }
        if (xsb != 0) return tiny - one;                            // x < -27 ln2 -> -1
    }

    // argument reduction
    if (hx > 0x3eb17218u) {             // |x| > 0.5 ln2
        if (hx < 0x3F851592u) {         // |x| < 1.5 ln2
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo;  k = 1; }
            else          { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int32_t)(invln2 * x + ((xsb == 0) ? 0.5f : -0.5f));
            t = (float)k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x33000000u) {      // |x| < 2^-25
        t = huge + x;
        return x - (t - (huge + x));
    } else {
        k = 0;
    }

    // x is now in the primary range
    hfx = 0.5f * x;
    hxs = x * hfx;
    r1 = one + hxs * (Q1 + hxs * (Q2 + hxs * (Q3 + hxs * (Q4 + hxs * Q5))));
    t = 3.0f - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0f - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5f * (x - e) - 0.5f;
    if (k == 1) {
        if (x < -0.25f) return -2.0f * (e - (x + 0.5f));
        return one + 2.0f * (x - e);
    }
    if (k <= -2 || k > 56) {            // suffices to return exp(x) - 1
        y = one - (e - x);
        y = u2f(f2u(y) + ((uint32_t)k << 23));
        return y - one;
    }
    if (k < 23) {
        t = u2f(0x3f800000u - (0x1000000u >> k));   // 1 - 2^-k
        y = t - (e - x);
        y = u2f(f2u(y) + ((uint32_t)k << 23));
    } else {
        t = u2f((uint32_t)(0x7f - k) << 23);        // 2^-k
        y = x - (e + t);
        y += one;
        y = u2f(f2u(y) + ((uint32_t)k << 23));
    }
    return y;
}

// tanhf following fdlibm s_tanhf.c.
ZM_HD float tanhf_fdlibm(float x)
{
    const float one = 1.0f, two = 2.0f, tiny = 1.0e-30f;
    const uint32_t jx = f2u(x);
    const uint32_t ix = jx & 0x7fffffffu;
    const bool neg = (jx >> 31) != 0;
    float t, z;

    if (ix >= 0x7f800000u) {            // inf or NaN
        if (!neg) return one / x + one; // tanh(+inf) = 1, NaN stays NaN
        return one / x - one;
    }
    if (ix < 0x41b00000u) {             // |x| < 22
        if (ix == 0) return x;          // +-0
        if (ix < 0x24000000u) return x * (one + x);   // |x| < 2^-55
        const float ax = u2f(ix);
        if (ix >= 0x3f800000u) {        // |x| >= 1
            t = expm1f_fdlibm(two * ax);
            z = one - two / (t + two);
        } else {
            t = expm1f_fdlibm(-two * ax);
            z = -t / (t + two);
        }
    } else {
        z = one - tiny;                 // |x| >= 22: 1 (inexact)
    }
    return neg ? -z : z;
}

// Quotient a / b for the two divisions inside tanhf_simd.  On the device: reciprocal estimate,
// product, one correction of the quotient by its exact remainder (4 instructions against the 11
// of the IEEE sequence with its operand scaling and fix-up).  That sequence is not correctly
// rounded for every pair of operands, but it is for every pair tanhf_simd feeds it (divisors in
// [5, 7] and [1, 2^30], no overflow, no underflow of the remainder): the kernel's results equal
// the host library's on all 2^32 arguments (tests/test_exhaustive_device.py).  The host build
// divides; it checks everything but this sequence.
ZM_HD float div_tanh(float a, float b)
{
#if defined(__HIP_DEVICE_COMPILE__) && !defined(ZMATH_EXACT_DIVISION)
    const float r = __builtin_amdgcn_rcpf(b);
    const float q = a * r;
    const float rem = __builtin_fmaf(-b, q, a);
    return __builtin_fmaf(rem, r, q);
#else
    return a / b;
#endif
}

// The same quotient for the other restated functions, and a square root in the same spirit
// (reciprocal square root estimate, one correction by the exact remainder; the argument must be
// positive and normal).  Each use is covered by the device check over every f32 bit pattern of
// the function it sits in; the host build divides and calls sqrtf.
ZM_HD float div_fast(float a, float b) { return div_tanh(a, b); }
ZM_HD float sqrt_fast(float t)
{
#if defined(__HIP_DEVICE_COMPILE__) && !defined(ZMATH_EXACT_DIVISION)
    const float y = __builtin_amdgcn_rsqf(t);
    const float s = t * y;
    const float h = 0.5f * y;
    const float r = __builtin_fmaf(-s, s, t);
    return __builtin_fmaf(r, h, s);
#else
    return __builtin_sqrtf(t);
#endif
}

// The same tanh, restructured for 64-wide SIMD execution: one path through the argument
// reduction, the rational core and ONE division pair for every lane, the per-k tails computed
// side by side and selected, so that a wavefront whose lanes hold |x| on both sides of 1 and
// different k does not execute the branches of tanhf_fdlibm one after another.  The results are
// tanhf_fdlibm's and the host libm's on every f32 bit pattern (tests/native/zmath_host_check.cpp
// on the host, tests/test_exhaustive_device.py on the device).
//
// The kernel is bound by its vector instructions (about 0.4 us per instruction and element on
// 2^24 elements), so the count is what matters.  Two kinds of savings.  Rewrites that perform
// fdlibm's operations on fdlibm's operands:
//   * hi = a - k*ln2_hi is one fused multiply-add: k*ln2_hi is exact (ln2_hi ends in 7 zero bits,
//     |k| < 64), so fusing does not change the rounding;
//   * the special cases |a| < 2^-25 (expm1 returns a) and |x| < 2^-55 (tanh returns x*(1+x)) need
//     no select: the k = 0 formula returns a there (its correction term is below half a unit in
//     the last place), and -a/(a+2) is then |x| exactly;
//   * k == 0: the correction c is 0, so e1 equals xr*e - hxs and the tail xr - (xr*e - hxs) is
//     -(e1 - xr): no arithmetic of its own;
//   * k == -1: 0.5*(xr - e1) - 0.5 = -0.5*(e1 - xr) - 0.5 shares e1 - xr with the other tails, and
//     is one fused multiply-add (the product is exact);
//   * k <= -2 and 2 <= k < 23 are one formula, A - (e1 - xr) scaled by 2^k, with A = 1 (and a
//     final - 1) or A = 1 - 2^-k; which of the two is decided by |x| >= 1 alone (then k >= 3,
//     else k <= 0), and the bit pattern that builds 1 - 2^-k is 1 for the negative k;
//   * |x| >= 9.02: 2/(expm1(2|x|) + 2) is below 2^-25 and vanishes against 1, so any large em1
//     gives the result 1 (fdlibm takes its k > 56 tail and its |x| >= 22 exit for this);
//     everything rare (k >= 23, i.e. |x| >= 7.8, and non-finite x) sits behind one test;
//   * the sign goes back with one bit operation.
// And departures from fdlibm's operation order whose only justification is the exhaustive check
// (each was tried alone and together over all 2^32 arguments of tanh and of the sigmoid; fusing any
// other multiply-add of the core changes between 15 and 17 526 results):
//   * k is a/ln2 rounded to nearest-even in one fused step instead of trunc(a/ln2 +- 0.5) with the
//     |a| <= 0.5 ln2 exception;
//   * four of the five Horner steps of the polynomial are fused multiply-adds.
// The core works on a2 = 2|x| (the sigmoid has it for free: tanh(x/2) needs a2 = |x|) and takes the
// sign and the NaN payload from `x`.
//
// Two constants meet a second constant in a fused multiply-add, and one instruction holds only one
// literal: the other has to sit in a vector register.  Left to the compiler it is written there
// again for every element; a kernel pins the pair once per thread (TanhRegs::pin) and passes it in.
struct TanhRegs {
    float magic = 12582912.0f;               // 1.5 * 2^23: adding it rounds to an integer
    float q4 = 4.0082177e-06f;               // 0x36867e54, the polynomial's fourth coefficient
    ZM_HD void pin()
    {
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("" : "+v"(magic), "+v"(q4));
#endif
    }
};

ZM_HD float tanhf_simd_core(float a2, float x, const TanhRegs &rg = TanhRegs())
{
    const float one = 1.0f, two = 2.0f;
    const float ln2_hi = u2f(0x3f317180u), ln2_lo = u2f(0x3717f7d1u), invln2 = u2f(0x3fb8aa3bu);
    const float Q1 = u2f(0xbd088889u), Q2 = u2f(0x3ad00d01u), Q3 = u2f(0xb8a670cdu),
                Q5 = u2f(0xb457edbbu);
    const bool big = a2 >= two;              // |x| >= 1: expm1(+2|x|), else expm1(-2|x|)
    const float a = big ? a2 : -a2;

    // expm1(a), a in (-2, 0] or [2, 44).  fdlibm takes k = trunc(a/ln2 +- 0.5), and 0 when |a| <= 0.5 ln2;
    // here k is a/ln2 rounded to the nearest integer by adding 1.5 * 2^23 in one fused step: the sum's
    // low mantissa bits are k (as a two's complement number), and subtracting the constant again
    // gives k as a float.  The two choices of k differ on a few ties, where either reduction gives
    // the same final bits.
    const float tkm = __builtin_fmaf(invln2, a, rg.magic);
    const float tk = tkm - rg.magic;
    const uint32_t kb = f2u(tkm);            // 0x4b400000 + k: only used where the upper bits fall out
    const int32_t k = (int32_t)(kb - 0x4b400000u);
#if defined(__HIP_DEVICE_COMPILE__)
    const float hi = __builtin_fmaf(-tk, ln2_hi, a);
#else
    const float hi = a - tk * ln2_hi;        // the product is exact: same value
#endif
    const float lo = tk * ln2_lo;
    const float xr = hi - lo;
    const float c = (hi - xr) - lo;

    const float hfx = 0.5f * xr;
    const float hxs = xr * hfx;
    // four of the five steps of the polynomial are fused: their rounding differences stay below
    // what reaches r1 on every argument (the last one, 1 + hxs * s, has to round twice)
    float sp = __builtin_fmaf(hxs, Q5, rg.q4);
    sp = __builtin_fmaf(hxs, sp, Q3);
    sp = __builtin_fmaf(hxs, sp, Q2);
    sp = __builtin_fmaf(hxs, sp, Q1);
    const float r1 = one + hxs * sp;
    const float t = 3.0f - r1 * hfx;
    const float e = hxs * div_tanh(r1 - t, 6.0f - xr * t);

    float e1 = xr * (e - c) - c;
    e1 -= hxs;
    const float d = e1 - xr;
    // k == 0: c is 0, so e1 is xr*e - hxs and fdlibm's xr - (xr*e - hxs) is -d
#if defined(__HIP_DEVICE_COMPILE__)
    const float mneg1 = __builtin_fmaf(-0.5f, d, -0.5f); // k == -1; -0.5*d is exact: fusing changes nothing
#else
    const float mneg1 = -0.5f * d - 0.5f;
#endif
    // |x| >= 1 has k >= 3: (1 - 2^-k) - d, scaled by 2^k.  |x| < 1 has k in {-3 .. 0}: (1 - d) scaled,
    // minus 1 -- and the shift count (k & 31) >= 29 leaves nothing of 2^24, so tt is already 1 there
    const float tt = u2f(0x3f800000u - (0x1000000u >> (kb & 31)));
    const float y = tt - d;
    const float ys = u2f(f2u(y) + (kb << 23));
    float em1 = big ? ys : ys - one;
    em1 = (kb == 0x4b3fffffu) ? mneg1 : em1;             // k == -1
    em1 = (kb == 0x4b400000u) ? -d : em1;                // k == 0
    if (!(a2 < 15.0f)) {                                 // |x| >= 7.5 (rare), or NaN
        if (k >= 23) {                                   // 2^-k no longer fits next to 1
            const float t2 = __builtin_ldexpf(one, -k);  // (the scalings are spelled differently from the one
            float y2 = xr - (e1 + t2);                   //  above so that it stays a single shift-and-add)
            y2 += one;
            em1 = __builtin_ldexpf(y2, k);
        }
        if (a2 >= u2f(0x419051ecu)) em1 = u2f(0x4e800000u);   // |x| >= 9.02: the result is 1 for any large em1
        if (a2 != a2) em1 = x;                           // NaN stays NaN
    }
    // |x| >= 1: 1 - 2/(t+2);  |x| < 1: -t/(t+2) = -(t/(t+2))
    const float q = div_tanh(big ? two : em1, em1 + two);
    const float z = big ? one - q : -q;
    return u2f((f2u(z) & 0x7fffffffu) | (f2u(x) & 0x80000000u));
}

ZM_HD float tanhf_simd(float x, const TanhRegs &rg = TanhRegs())
{
    const float ax = u2f(f2u(x) & 0x7fffffffu);
    return tanhf_simd_core(ax + ax, x, rg);
}

// ---- f32 exp and log: the table-driven routines glibc ships since 2.27 (from ARM's optimized routines) ----
// expf:  x*N/ln2 = k + r, N = 32;  exp(x) = 2^(k/N) * 2^(r/N) ~ T[k % N] * 2^(k / N) * (C0 r^3 + C1 r^2 + C2 r + 1),
//        evaluated in double and rounded once to float.
// logf:  x = 2^k z, z in [0x3f330000, 2*0x3f330000) split into N = 16 intervals with centre c;
//        log(x) = log1p(z/c - 1) + log(c) + k ln2, a cubic in r = z * (1/c) - 1, in double.
// The reduction r = fma(InvLn2N, x, -k) is the fused form that the x86-64 build with FMA (the one a
// CPU with FMA selects at run time) produces; with it the results equal the host libm's on every
// f32 bit pattern (the non-fused form differs on 2 of the 2^32 inputs of expf, by one ulp).
// Checked exhaustively by tests/native/zmath_host_check.cpp.

#define ZM_EXP2F_TAB                                                                                        \
    { 0x3ff0000000000000ull, 0x3fefd9b0d3158574ull, 0x3fefb5586cf9890full, 0x3fef9301d0125b51ull,           \
      0x3fef72b83c7d517bull, 0x3fef54873168b9aaull, 0x3fef387a6e756238ull, 0x3fef1e9df51fdee1ull,           \
      0x3fef06fe0a31b715ull, 0x3feef1a7373aa9cbull, 0x3feedea64c123422ull, 0x3feece086061892dull,           \
      0x3feebfdad5362a27ull, 0x3feeb42b569d4f82ull, 0x3feeab07dd485429ull, 0x3feea47eb03a5585ull,           \
      0x3feea09e667f3bcdull, 0x3fee9f75e8ec5f74ull, 0x3feea11473eb0187ull, 0x3feea589994cce13ull,           \
      0x3feeace5422aa0dbull, 0x3feeb737b0cdc5e5ull, 0x3feec49182a3f090ull, 0x3feed503b23e255dull,           \
      0x3feee89f995ad3adull, 0x3feeff76f2fb5e47ull, 0x3fef199bdd85529cull, 0x3fef3720dcef9069ull,           \
      0x3fef5818dcfba487ull, 0x3fef7c97337b9b5full, 0x3fefa4afa2a490daull, 0x3fefd0765b6e4540ull }
// {1/c, log(c)} per interval
#define ZM_LOGF_TAB                                                                                         \
    { 0x1.661ec79f8f3bep+0, -0x1.57bf7808caadep-2, 0x1.571ed4aaf883dp+0, -0x1.2bef0a7c06ddbp-2,             \
      0x1.49539f0f010bp+0, -0x1.01eae7f513a67p-2, 0x1.3c995b0b80385p+0, -0x1.b31d8a68224e9p-3,              \
      0x1.30d190c8864a5p+0, -0x1.6574f0ac07758p-3, 0x1.25e227b0b8eap+0, -0x1.1aa2bc79c81p-3,                \
      0x1.1bb4a4a1a343fp+0, -0x1.a4e76ce8c0e5ep-4, 0x1.12358f08ae5bap+0, -0x1.1973c5a611cccp-4,             \
      0x1.0953f419900a7p+0, -0x1.252f438e10c1ep-5, 0x1p+0, 0x0p+0,                                          \
      0x1.e608cfd9a47acp-1, 0x1.aa5aa5df25984p-5, 0x1.ca4b31f026aap-1, 0x1.c5e53aa362eb4p-4,                \
      0x1.b2036576afce6p-1, 0x1.526e57720db08p-3, 0x1.9c2d163a1aa2dp-1, 0x1.bc2860d22477p-3,                \
      0x1.886e6037841edp-1, 0x1.1058bc8a07ee1p-2, 0x1.767dcf5534862p-1, 0x1.4043057b6ee09p-2 }

// powf's {1/c, log2(c)} per interval (same centres as logf's)
#define ZM_POWF_LOG2_TAB                                                                                    \
    { 0x1.661ec79f8f3bep+0, -0x1.efec65b963019p-2, 0x1.571ed4aaf883dp+0, -0x1.b0b6832d4fca4p-2,             \
      0x1.49539f0f010bp+0, -0x1.7418b0a1fb77bp-2, 0x1.3c995b0b80385p+0, -0x1.39de91a6dcf7bp-2,              \
      0x1.30d190c8864a5p+0, -0x1.01d9bf3f2b631p-2, 0x1.25e227b0b8eap+0, -0x1.97c1d1b3b7afp-3,               \
      0x1.1bb4a4a1a343fp+0, -0x1.2f9e393af3c9fp-3, 0x1.12358f08ae5bap+0, -0x1.960cbbf788d5cp-4,             \
      0x1.0953f419900a7p+0, -0x1.a6f9db6475fcep-5, 0x1p+0, 0x0p+0,                                          \
      0x1.e608cfd9a47acp-1, 0x1.338ca9f24f53dp-4, 0x1.ca4b31f026aap-1, 0x1.476a9543891bap-3,                \
      0x1.b2036576afce6p-1, 0x1.e840b4ac4e4d2p-3, 0x1.9c2d163a1aa2dp-1, 0x1.40645f0c6651cp-2,               \
      0x1.886e6037841edp-1, 0x1.88e9c2c1b9ff8p-2, 0x1.767dcf5534862p-1, 0x1.ce0a44eb17bccp-2 }

static const uint64_t kExp2fTabHost[32] = ZM_EXP2F_TAB;
static const double kLogfTabHost[32] = ZM_LOGF_TAB;
static const double kPowfLog2TabHost[32] = ZM_POWF_LOG2_TAB;
#if defined(__HIPCC__)
static __device__ const uint64_t kExp2fTabDev[32] = ZM_EXP2F_TAB;
static __device__ const double kLogfTabDev[32] = ZM_LOGF_TAB;
static __device__ const double kPowfLog2TabDev[32] = ZM_POWF_LOG2_TAB;
#endif

// the tables as seen from the code being compiled (device: global memory; kernels that evaluate
// many elements copy them into LDS first, a gather from global memory costs a tag lookup per lane)
ZM_HD const uint64_t *exp2f_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return kExp2fTabDev;
#else
    return kExp2fTabHost;
#endif
}
ZM_HD const double *logf_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return kLogfTabDev;
#else
    return kLogfTabHost;
#endif
}

ZM_HD const double *powf_log2_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return kPowfLog2TabDev;
#else
    return kPowfLog2TabHost;
#endif
}

ZM_HD uint64_t d2u(double d);
ZM_HD double u2d(uint64_t u);

// The double constants of expf / logf as data (see SinCosCoef): a kernel hands them over in its
// argument, every other caller takes the defaults.
struct ExpfCoef {
    double inv_ln2n = 0x1.71547652b82fep+0 * 32, shift = 0x1.8p+52;
    double c0 = 0x1.c6af84b912394p-5 / 32 / 32 / 32, c1 = 0x1.ebfce50fac4f3p-3 / 32 / 32, c2 = 0x1.62e42ff0c52d6p-1 / 32;
};
struct LogfCoef {
    double a0 = -0x1.00ea348b88334p-2, a1 = 0x1.5575b0be00b6ap-2, a2 = -0x1.ffffef20a4123p-2;
    double ln2 = 0x1.62e42fefa39efp-1;
};

ZM_HD float expf_glibc(float x, const uint64_t *tab, const ExpfCoef &k = ExpfCoef())
{
    const uint32_t ux = f2u(x);
    const uint32_t abstop = (ux >> 20) & 0x7ffu;
    if (abstop >= (0x42b00000u >> 20)) {                 // |x| >= 88 or NaN
        if (ux == 0xff800000u) return 0.0f;              // -inf
        if (abstop >= (0x7f800000u >> 20)) return x + x; // +inf, NaN
        if (x > 0x1.62e42ep6f) return u2f(0x7f800000u);  // overflow
        if (x < -0x1.9fe368p6f) return 0.0f;             // underflow
    }
    const double xd = (double)x;
    const double z = k.inv_ln2n * xd;
    double kd = z + k.shift;
    const uint64_t ki = d2u(kd);
    kd -= k.shift;
    const double r = __builtin_fma(k.inv_ln2n, xd, -kd);
    const uint64_t t = tab[ki % 32] + (ki << (52 - 5));
    const double s = u2d(t);
    const double p = __builtin_fma(k.c0, r, k.c1);
    const double r2 = r * r;
    double y = __builtin_fma(k.c2, r, 1.0);
    y = __builtin_fma(p, r2, y);
    y = y * s;
    return (float)y;
}

// The main path alone, for callers whose argument cannot overflow or underflow (|x| < 87): the
// operations of expf_glibc on such an argument, nothing else.
ZM_HD float expf_glibc_core(float x, const uint64_t *tab, const ExpfCoef &k = ExpfCoef())
{
    const double xd = (double)x;
    const double z = k.inv_ln2n * xd;
    double kd = z + k.shift;
    const uint64_t ki = d2u(kd);
    kd -= k.shift;
    const double r = __builtin_fma(k.inv_ln2n, xd, -kd);
    const uint64_t t = tab[ki % 32] + (ki << (52 - 5));
    const double s = u2d(t);
    const double p = __builtin_fma(k.c0, r, k.c1);
    const double r2 = r * r;
    double y = __builtin_fma(k.c2, r, 1.0);
    y = __builtin_fma(p, r2, y);
    y = y * s;
    return (float)y;
}

// The same expf without a branch, for kernels whose scalar unit is the busy one (a branch per element
// is half a dozen scalar instructions): the main path runs on any bit pattern (the table index is
// taken modulo the table size; a NaN stays a NaN), overflow and underflow are two selects.  Same
// results as expf_glibc except for the payload of a NaN.
ZM_HD float expf_glibc_flat(float x, const uint64_t *tab, const ExpfCoef &k = ExpfCoef())
{
    const double xd = (double)x;
    const double z = k.inv_ln2n * xd;
    double kd = z + k.shift;
    const uint64_t ki = d2u(kd);
    kd -= k.shift;
    const double r = __builtin_fma(k.inv_ln2n, xd, -kd);
    const uint64_t t = tab[ki % 32] + (ki << (52 - 5));
    const double s = u2d(t);
    const double p = __builtin_fma(k.c0, r, k.c1);
    const double r2 = r * r;
    double y = __builtin_fma(k.c2, r, 1.0);
    y = __builtin_fma(p, r2, y);
    y = y * s;
    float res = (float)y;
    res = (x > 0x1.62e42ep6f) ? u2f(0x7f800000u) : res;  // overflow, +inf
    res = (x < -0x1.9fe368p6f) ? 0.0f : res;             // underflow, -inf
    return res;
}

// logf: the routine with its special cases, and below it the main path as straight-line code for
// positive normal arguments, which hands zero, negative, subnormal, infinite and NaN arguments back
ZM_HD float logf_glibc_full(float x, const double *tab)
{
    const double A0 = -0x1.00ea348b88334p-2, A1 = 0x1.5575b0be00b6ap-2, A2 = -0x1.ffffef20a4123p-2;
    const double Ln2 = 0x1.62e42fefa39efp-1;
    uint32_t ix = f2u(x);
    if (ix == 0x3f800000u) return 0.0f;
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u) { // x < 2^-126, inf or NaN
        if (ix * 2 == 0) return u2f(0xff800000u);        // log(+-0) = -inf
        if (ix == 0x7f800000u) return x;                 // log(inf) = inf
        if ((ix & 0x80000000u) || ix * 2 >= 0xff000000u) return (x - x) * u2f(0x7f800000u);   // NaN: the sources' (x - x) / (x - x) without the division
        ix = f2u(x * 0x1p23f);                           // subnormal: normalise
        ix -= 23u << 23;
    }
    const uint32_t tmp = ix - 0x3f330000u;
    const uint32_t i = (tmp >> (23 - 4)) % 16;
    const int32_t k = (int32_t)tmp >> 23;
    const uint32_t iz = ix - (tmp & (0x1ffu << 23));
    const double invc = tab[2 * i], logc = tab[2 * i + 1];
    const double z = (double)u2f(iz);
    const double r = __builtin_fma(z, invc, -1.0);
    const double y0 = __builtin_fma((double)k, Ln2, logc);
    const double r2 = r * r;
    double y = __builtin_fma(A1, r, A2);
    y = __builtin_fma(A0, r2, y);
    y = __builtin_fma(y, r2, y0 + r);
    return (float)y;
}

ZM_RARE float logf_rare(float x, const double *tab) { return logf_glibc_full(x, tab); }

ZM_HD float logf_glibc(float x, const double *tab, const LogfCoef &c = LogfCoef())
{
    const uint32_t ix = f2u(x);
    const uint32_t tmp = ix - 0x3f330000u;
    const uint32_t i = (tmp >> (23 - 4)) % 16;
    const int32_t k = (int32_t)tmp >> 23;
    const uint32_t iz = ix - (tmp & (0x1ffu << 23));
    const double invc = tab[2 * i], logc = tab[2 * i + 1];
    const double z = (double)u2f(iz);
    const double r = __builtin_fma(z, invc, -1.0);
    const double y0 = __builtin_fma((double)k, c.ln2, logc);
    const double r2 = r * r;
    double y = __builtin_fma(c.a1, r, c.a2);
    y = __builtin_fma(c.a0, r2, y);
    y = __builtin_fma(y, r2, y0 + r);
    if (__builtin_expect(ix - 0x00800000u >= 0x7f800000u - 0x00800000u, 0)) return logf_rare(x, tab);
    return (float)y;                                     // (x = 1 gives +0 here as well: r and y0 are 0)
}

// powf (glibc's e_powf.c, same origin): x^y = 2^(y log2 x); log2 x as a quartic in r = z/c - 1 around
// the 16 interval centres, the product y log2(x) and the 2^ step (exp2f's 32-entry table and cubic)
// all in double, rounded once to float.  Results equal the host libm's with the fused and with
// the unfused evaluation on every sampled input (tests/native/zmath_host_check.cpp).
// 0 = not an integer, 1 = odd integer, 2 = even integer
ZM_HD int powf_checkint(uint32_t iy)
{
    const int e = (int)(iy >> 23 & 0xffu);
    if (e < 0x7f) return 0;
    if (e > 0x7f + 23) return 2;
    if (iy & ((1u << (0x7f + 23 - e)) - 1u)) return 0;
    if (iy & (1u << (0x7f + 23 - e))) return 1;
    return 2;
}
ZM_HD bool powf_zeroinfnan(uint32_t i) { return 2u * i - 1u >= 2u * 0x7f800000u - 1u; }
ZM_HD bool powf_signaling(uint32_t i) { return 2u * (i ^ 0x00400000u) > 2u * 0x7fc00000u; }

ZM_HD float powf_glibc_full(float x, float y, const uint64_t *etab, const double *ltab)
{
    const double A0 = 0x1.27616c9496e0bp-2, A1 = -0x1.71969a075c67ap-2, A2 = 0x1.ec70a6ca7baddp-2,
                 A3 = -0x1.7154748bef6c8p-1, A4 = 0x1.71547652ab82bp0;
    const double C0 = 0x1.c6af84b912394p-5, C1 = 0x1.ebfce50fac4f3p-3, C2 = 0x1.62e42ff0c52d6p-1;
    const double Shift = 0x1.8p+52 / 32;
    uint32_t sign_bias = 0;
    uint32_t ix = f2u(x);
    const uint32_t iy = f2u(y);
    if (ix - 0x00800000u >= 0x7f800000u - 0x00800000u || powf_zeroinfnan(iy)) {
        // x < 2^-126, inf or NaN; or y zero, inf or NaN
        if (powf_zeroinfnan(iy)) {
            if (2u * iy == 0) return powf_signaling(ix) ? x + y : 1.0f;
            if (ix == 0x3f800000u) return powf_signaling(iy) ? x + y : 1.0f;
            if (2u * ix > 2u * 0x7f800000u || 2u * iy > 2u * 0x7f800000u) return x + y;
            if (2u * ix == 2u * 0x3f800000u) return 1.0f;
            if ((2u * ix < 2u * 0x3f800000u) == !(iy & 0x80000000u)) return 0.0f;   // |x|<1, y=inf or |x|>1, y=-inf
            return y * y;
        }
        if (powf_zeroinfnan(ix)) {
            float x2 = x * x;
            if ((ix & 0x80000000u) && powf_checkint(iy) == 1) x2 = -x2;
            return (iy & 0x80000000u) ? 1.0f / x2 : x2;
        }
        if (ix & 0x80000000u) {                          // finite x < 0
            const int yint = powf_checkint(iy);
            if (yint == 0) return (x - x) * u2f(0x7f800000u);   // NaN: the sources' (x - x) / (x - x) without the division
            if (yint == 1) sign_bias = 1u << (5 + 11);
            ix &= 0x7fffffffu;
        }
        if (ix < 0x00800000u) {                          // subnormal: normalise
            ix = f2u(x * 0x1p23f);
            ix &= 0x7fffffffu;
            ix -= 23u << 23;
        }
    }
    // log2(x) = log1p(z/c - 1)/ln2 + log2(c) + k
    const uint32_t tmp = ix - 0x3f330000u;
    const uint32_t i = (tmp >> (23 - 4)) % 16;
    const uint32_t top = tmp & 0xff800000u;
    const uint32_t iz = ix - top;
    const int32_t k = (int32_t)top >> 23;
    const double invc = ltab[2 * i], logc = ltab[2 * i + 1];
    const double z = (double)u2f(iz);
    const double r = __builtin_fma(z, invc, -1.0);
    const double y0 = logc + (double)k;
    const double r2 = r * r;
    double yy = __builtin_fma(A0, r, A1);
    const double p = __builtin_fma(A2, r, A3);
    const double r4 = r2 * r2;
    double q = __builtin_fma(A4, r, y0);
    q = __builtin_fma(p, r2, q);
    yy = __builtin_fma(yy, r4, q);
    const double ylogx = (double)y * yy;                 // cannot overflow: y is single precision
    if ((d2u(ylogx) >> 47 & 0xffffu) >= (d2u(126.0) >> 47)) {   // |y log2 x| >= 126
        if (ylogx > 0x1.fffffffd1d571p+6) return u2f(sign_bias ? 0xff800000u : 0x7f800000u);
        if (ylogx <= -150.0) return u2f(sign_bias ? 0x80000000u : 0u);
    }
    // 2^(y log2 x): x' = k/N + r', |r'| <= 1/(2N)
    double kd = ylogx + Shift;
    const uint64_t ki = d2u(kd);
    kd -= Shift;
    const double rr = ylogx - kd;
    uint64_t t = etab[ki % 32];
    t += (ki + sign_bias) << (52 - 5);
    const double s = u2d(t);
    const double zz = __builtin_fma(C0, rr, C1);
    const double rr2 = rr * rr;
    double out = __builtin_fma(C2, rr, 1.0);
    out = __builtin_fma(zz, rr2, out);
    out = out * s;
    return (float)out;
}

// The constants of the main path as data (see SinCosCoef).
struct PowCoef {
    double a0 = 0x1.27616c9496e0bp-2, a1 = -0x1.71969a075c67ap-2, a2 = 0x1.ec70a6ca7baddp-2,
           a3 = -0x1.7154748bef6c8p-1, a4 = 0x1.71547652ab82bp0;
    double c0 = 0x1.c6af84b912394p-5, c1 = 0x1.ebfce50fac4f3p-3, c2 = 0x1.62e42ff0c52d6p-1;
    double shift = 0x1.8p+52 / 32;
};

// powf as the kernels call it: the main path of powf_glibc_full as straight-line code (positive
// normal x, finite non-zero y, |y log2 x| < 126: no special case applies, no sign to carry), and
// one branch to the full routine for everything else.
ZM_RARE float powf_rare(float x, float y, const uint64_t *etab, const double *ltab) { return powf_glibc_full(x, y, etab, ltab); }

ZM_HD float powf_glibc(float x, float y, const uint64_t *etab, const double *ltab, const PowCoef &k = PowCoef())
{
    const uint32_t ix = f2u(x), iy = f2u(y);
    // (the main path runs on any bit pattern without harm: its table indices are taken modulo the
    // table sizes; whether its result stands is decided once, at the end)
    const bool special = ix - 0x00800000u >= 0x7f800000u - 0x00800000u || powf_zeroinfnan(iy);
    const uint32_t tmp = ix - 0x3f330000u;
    const uint32_t i = (tmp >> (23 - 4)) % 16;
    const uint32_t top = tmp & 0xff800000u;
    const uint32_t iz = ix - top;
    const int32_t kk = (int32_t)top >> 23;
    const double invc = ltab[2 * i], logc = ltab[2 * i + 1];
    const double z = (double)u2f(iz);
    const double r = __builtin_fma(z, invc, -1.0);
    const double y0 = logc + (double)kk;
    const double r2 = r * r;
    double yy = __builtin_fma(k.a0, r, k.a1);
    const double p = __builtin_fma(k.a2, r, k.a3);
    const double r4 = r2 * r2;
    double q = __builtin_fma(k.a4, r, y0);
    q = __builtin_fma(p, r2, q);
    yy = __builtin_fma(yy, r4, q);
    const double ylogx = (double)y * yy;
    const bool wide = (d2u(ylogx) >> 47 & 0xffffu) >= (d2u(126.0) >> 47);   // |y log2 x| >= 126, or NaN
    double kd = ylogx + k.shift;
    const uint64_t ki = d2u(kd);
    kd -= k.shift;
    const double rr = ylogx - kd;
    uint64_t t = etab[ki % 32];
    t += ki << (52 - 5);
    const double sc = u2d(t);
    const double zz = __builtin_fma(k.c0, rr, k.c1);
    const double rr2 = rr * rr;
    double out = __builtin_fma(k.c2, rr, 1.0);
    out = __builtin_fma(zz, rr2, out);
    out = out * sc;
    if (__builtin_expect(special || wide, 0)) return powf_rare(x, y, etab, ltab);
    return (float)out;
}

// sinhf / coshf (fdlibm e_sinhf.c / e_coshf.c as glibc 2.35 ships them): expm1f below 22, expf above,
// the argument halved where exp would overflow.  `etab` is expf's table.
ZM_HD float sinhf_fdlibm(float x, const uint64_t *etab)
{
    const float one = 1.0f, shuge = 1.0e37f;
    const uint32_t jx = f2u(x);
    const uint32_t ix = jx & 0x7fffffffu;
    if (ix >= 0x7f800000u) return x + x;                 // inf, NaN
    const float h = (jx & 0x80000000u) ? -0.5f : 0.5f;
    const float ax = u2f(ix);
    if (ix < 0x41b00000u) {                              // |x| < 22
        if (ix < 0x31800000u) return x;                  // |x| < 2^-28
        const float t = expm1f_fdlibm(ax);
        if (ix < 0x3f800000u) return h * (2.0f * t - t * t / (t + one));
        return h * (t + t / (t + one));
    }
    if (ix < 0x42b17180u) return h * expf_glibc(ax, etab);   // |x| < log(FLT_MAX)
    if (ix <= 0x42b2d4fcu) {                             // up to the overflow threshold
        const float w = expf_glibc(0.5f * ax, etab);
        const float t = h * w;
        return t * w;
    }
    return x * shuge;                                    // overflow
}

ZM_HD float coshf_fdlibm(float x, const uint64_t *etab)
{
    const float one = 1.0f, half = 0.5f, huge = 1.0e30f;
    const uint32_t ix = f2u(x) & 0x7fffffffu;
    const float ax = u2f(ix);
    if (ix < 0x41b00000u) {                              // |x| < 22
        if (ix < 0x3eb17218u) {                          // |x| < 0.5 ln2: 1 + expm1^2 / (2 exp)
            if (ix < 0x24000000u) return one;
            const float t = expm1f_fdlibm(ax);
            const float w = one + t;
            return one + (t * t) / (w + w);
        }
        const float t = expf_glibc(ax, etab);
        return half * t + half / t;
    }
    if (ix < 0x42b17180u) return half * expf_glibc(ax, etab);
    if (ix <= 0x42b2d4fcu) {
        const float w = expf_glibc(half * ax, etab);
        const float t = half * w;
        return t * w;
    }
    if (ix >= 0x7f800000u) return x * x;                 // inf, NaN
    return huge * huge;                                  // overflow
}

// sinf / cosf (glibc's s_sinf.c / s_cosf.c with sincosf.h, from ARM's optimized routines), in double:
// |x| < pi/4 a polynomial; |x| < 120 one multiply-subtract reduction by pi/2 with the quadrant from a
// scaled float-to-int conversion; larger arguments a 32 x 96 bit fixed-point product with 4/pi.
// Every a + b*c is fused, as in the x86-64 build that CPUs with FMA select; with that the results
// equal the host libm's on all 2^32 inputs (the unfused form differs on 12 / 22 of them).
// 4/pi to 192 bits, 8 new bits per entry
#define ZM_INV_PIO4_TAB                                                                                     \
    { 0xa2u, 0xa2f9u, 0xa2f983u, 0xa2f9836eu, 0xf9836e4eu, 0x836e4e44u, 0x6e4e4415u, 0x4e441529u,           \
      0x441529fcu, 0x1529fc27u, 0x29fc2757u, 0xfc2757d1u, 0x2757d1f5u, 0x57d1f534u, 0xd1f534ddu,            \
      0xf534ddc0u, 0x34ddc0dbu, 0xddc0db62u, 0xc0db6295u, 0xdb629599u, 0x6295993cu, 0x95993c43u,            \
      0x993c4390u, 0x3c439041u }
static const uint32_t kInvPio4Host[24] = ZM_INV_PIO4_TAB;
#if defined(__HIPCC__)
static __device__ const uint32_t kInvPio4Dev[24] = ZM_INV_PIO4_TAB;
#endif
ZM_HD const uint32_t *inv_pio4_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return kInvPio4Dev;
#else
    return kInvPio4Host;
#endif
}

// sine polynomial for an even quadrant, cosine polynomial for an odd one; `neg` flips the cosine
ZM_HD float sincosf_poly(double x, double x2, bool neg, int n)
{
    if ((n & 1) == 0) {
        const double S1 = -0x1.555545995a603p-3, S2 = 0x1.1107605230bc4p-7, S3 = -0x1.994eb3774cf24p-13;
        const double x3 = x * x2;
        const double s1 = __builtin_fma(x2, S3, S2);
        const double x7 = x3 * x2;
        const double s = __builtin_fma(x3, S1, x);
        return (float)__builtin_fma(x7, s1, s);
    }
    const double sg = neg ? -1.0 : 1.0;
    const double C0 = sg, C1 = sg * -0x1.ffffffd0c621cp-2, C2 = sg * 0x1.55553e1068f19p-5,
                 C3 = sg * -0x1.6c087e89a359dp-10, C4 = sg * 0x1.99343027bf8c3p-16;
    const double x4 = x2 * x2;
    const double c2 = __builtin_fma(x2, C4, C3);
    const double c1 = __builtin_fma(x2, C1, C0);
    const double x6 = x4 * x2;
    const double c = __builtin_fma(x4, C2, c1);
    return (float)__builtin_fma(x6, c2, c);
}

// The constants of the common path as data: handed to a kernel as an argument they sit in scalar
// registers and feed the f64 operations directly (as literals each one is copied into a register
// pair before every use, two scalar instructions per constant and element).
struct SinCosCoef {
    double hpi_inv = 0x1.45F306DC9C883p+23, hpi = 0x1.921FB54442D18p0;
    double s1 = -0x1.555545995a603p-3, s2 = 0x1.1107605230bc4p-7, s3 = -0x1.994eb3774cf24p-13;
    double c1 = -0x1.ffffffd0c621cp-2, c2 = 0x1.55553e1068f19p-5, c3 = -0x1.6c087e89a359dp-10, c4 = 0x1.99343027bf8c3p-16;
};

// cosine = 0: sinf(y); cosine = 1: cosf(y)
ZM_HD float sincosf_glibc(float y, int cosine, const SinCosCoef &k = SinCosCoef())
{
    const double Pi63 = 0x1.921FB54442D18p-62;
    const uint32_t top = (f2u(y) >> 20) & 0x7ffu;
    if (top < (0x42f00000u >> 20)) {                     // |y| < 120
        // The sources branch off |y| < pi/4 (and |y| < 2^-12) first; the reduction below finds n = 0
        // there and leaves x alone, and the polynomials round to y resp. 1 below 2^-12, so one path
        // serves all three.  The signs (the sources multiply x by +-1 and the cosine coefficients by
        // +-1) are applied to the result instead: every operation is odd resp. even in them.
        double x = (double)y;
        const double r = x * k.hpi_inv;
        const int n = ((int32_t)r + 0x800000) >> 24;
        x = __builtin_fma(-(double)n, k.hpi, x);
        const double x2 = x * x;
        const bool odd = ((n ^ cosine) & 1) != 0;
        float res;
        if (!odd) {                                      // on |x|: a zero keeps its sign that way
            const double ax = __builtin_fabs(x);
            const double x3 = ax * x2;
            const double s1 = __builtin_fma(x2, k.s3, k.s2);
            const double x7 = x3 * x2;
            const double sv = __builtin_fma(x3, k.s1, ax);
            res = (float)__builtin_fma(x7, s1, sv);
        } else {
            const double x4 = x2 * x2;
            const double c2 = __builtin_fma(x2, k.c4, k.c3);
            const double c1 = __builtin_fma(x2, k.c1, 1.0);
            const double x6 = x4 * x2;
            const double c = __builtin_fma(x4, k.c2, c1);
            res = (float)__builtin_fma(x6, c2, c);
        }
        // sine polynomial: the sign of x, flipped in quadrants 1 and 2; cosine polynomial: negative in quadrants 2 and 3
        const uint32_t flip = odd ? (uint32_t)n >> 1 : (((uint32_t)n + 1u) >> 1) ^ (uint32_t)(d2u(x) >> 63);
        return u2f(f2u(res) ^ (flip << 31));
    }
    if (top < (0x7f800000u >> 20)) {
        uint32_t xi = f2u(y);
        const int sign = (int)(xi >> 31);
        const uint32_t *arr = inv_pio4_table() + ((xi >> 26) & 15u);
        const int shift = (int)((xi >> 23) & 7u);
        xi = (xi & 0xffffffu) | 0x800000u;
        xi <<= shift;
        uint64_t res0 = (uint64_t)(uint32_t)(xi * arr[0]);
        const uint64_t res1 = (uint64_t)xi * arr[4];
        const uint64_t res2 = (uint64_t)xi * arr[8];
        res0 = (res2 >> 32) | (res0 << 32);
        res0 += res1;
        const uint64_t q = (res0 + (1ull << 61)) >> 62;
        res0 -= q << 62;
        const double x = (double)(int64_t)res0 * Pi63;
        const int n = (int)q + sign;
        const double s = ((n & 3) == 1 || (n & 3) == 2) ? -1.0 : 1.0;
        return sincosf_poly(x * s, x * x, (n & 2) != 0, (int)q ^ cosine);
    }
    return (y - y) / (y - y);                            // inf, NaN
}
// tanf (glibc 2.35: s_tanf.c and k_tanf.c are fdlibm's float code; e_rem_pio2f.c hands them sincosf's
// argument reduction: the reduced argument in double, split into a float and the float remainder,
// and the quadrant).  These files have no FMA build: every product rounds, also the one of the
// reduction that sinf / cosf fuse.  Equal to the host libm on all 2^32 arguments.
//
// Restructured for 64-wide execution: one path through the reduction, the polynomial and ONE
// division for every lane (the sources branch three ways after the polynomial, and two of the
// branches divide).  What the sources decide beforehand folds into that path:
//   * |x| <= pi/4 (their call of the kernel on x itself): the reduction finds quadrant 0 there and
//     leaves x alone, with remainder 0;
//   * a reduced argument below 2^-13 in an even quadrant (they return it): the general formula does
//     too, x + (y + ...) with everything in the bracket below a quarter unit of x -- except that y can
//     be exactly half a unit, so the case keeps its select;
//   * x = 0 in an odd quadrant (1 / |x|) cannot occur: no float but 0 reduces to 0.
// |x| >= 120: |x| times 4/pi as a 32 x 96 bit fixed-point product.  Returns the remainder after the
// nearest multiple of pi/2 (in units of pi/2 2^-62, below 2^61 in magnitude) shifted left by one, with
// the parity of that multiple in bit 0.  Out of line: few tensors hold such arguments.
ZM_RARE int64_t tanf_reduce_large(uint32_t xi)
{
    const uint32_t *arr = inv_pio4_table() + ((xi >> 26) & 15u);
    const int shift = (int)((xi >> 23) & 7u);
    xi = (xi & 0xffffffu) | 0x800000u;
    xi <<= shift;
    uint64_t res0 = (uint64_t)(uint32_t)(xi * arr[0]);
    const uint64_t res1 = (uint64_t)xi * arr[4];
    const uint64_t res2 = (uint64_t)xi * arr[8];
    res0 = (res2 >> 32) | (res0 << 32);
    res0 += res1;
    const uint64_t q = (res0 + (1ull << 61)) >> 62;
    res0 -= q << 62;
    return (int64_t)(res0 << 1) | (int64_t)(q & 1u);
}
struct TanfCoef {
    double hpi_inv = 0x1.45F306DC9C883p+23, hpi = 0x1.921FB54442D18p0;
};
ZM_HD float tanf_glibc(float xf, const TanfCoef &k = TanfCoef())
{
    const float pio4 = 7.8539812565e-01f, pio4lo = 3.7748947079e-08f;
    const float T0 = 3.3333334327e-01f, T1 = 1.3333334029e-01f, T2 = 5.3968254477e-02f, T3 = 2.1869488060e-02f,
                T4 = 8.8632395491e-03f, T5 = 3.5920790397e-03f, T6 = 1.4562094584e-03f, T7 = 5.8804126456e-04f,
                T8 = 2.4646313977e-04f, T9 = 7.8179444245e-05f, T10 = 7.1407252108e-05f, T11 = -1.8558637748e-05f,
                T12 = 2.5907305826e-05f;
    const uint32_t top = (f2u(xf) >> 20) & 0x7ffu;
    double dx = (double)xf;
    int n;
    if (__builtin_expect(top < (0x42f00000u >> 20), 1)) {        // |x| < 120
        const double r = dx * k.hpi_inv;
        n = ((int32_t)r + 0x800000) >> 24;
        dx = dx - (double)n * k.hpi;
    } else if (top < (0x7f800000u >> 20)) {
        const int64_t packed = tanf_reduce_large(f2u(xf));
        dx = (double)(packed >> 1) * 0x1.921FB54442D18p-62;
        if (f2u(xf) >> 31) dx = -dx;
        n = (int)(packed & 1);                           // only the quadrant's parity matters, and -q has q's
    } else {
        return (xf - xf) * u2f(0x7f800000u);             // inf, NaN: the sources' x - x
    }
    const float y0 = (float)dx;
    const float y1 = (float)(dx - (double)y0);
    const bool odd = (n & 1) != 0;
    const float fiy = odd ? -1.0f : 1.0f;                // the sources' iy

    const uint32_t hx = f2u(y0);
    const uint32_t ix = hx & 0x7fffffffu;
    const bool big = ix >= 0x3f2ca140u;                  // |y0| >= 0.6744: tan(pi/4 - |y0|) and the angle sum
    const bool tiny = ix < 0x39000000u;                  // |y0| < 2^-13
    const uint32_t sgn = hx & 0x80000000u;
    float x = y0, y = y1;
    if (big) {
        const float z0 = pio4 - u2f(ix);
        const float w0 = pio4lo - u2f(f2u(y1) ^ sgn);
        x = z0 + w0;
        y = 0.0f;
    }
    const float z = x * x;
    const float w2 = z * z;
    // the two innermost Horner steps of the first polynomial and the three innermost of the second are
    // fused: that changes none of the 2^32 results (each was tried alone, then all five together;
    // fusing any other step changes between 36 and 22 535 338 of them)
    float r = __builtin_fmaf(w2, __builtin_fmaf(w2, T11, T9), T7);
    r = T1 + w2 * (T3 + w2 * (T5 + w2 * r));
    float v = __builtin_fmaf(w2, __builtin_fmaf(w2, __builtin_fmaf(w2, T12, T10), T8), T6);
    v = z * (T2 + w2 * (T4 + w2 * v));
    const float s = z * x;
    r = y + z * (s * (r + v) + y);
    r += T0 * s;
    const float w = x + r;
    // the one quotient: w w / (w + iy) of the first branch, -1 / w of an odd quadrant (-1 / y0 below 2^-13)
    const float num = big ? w * w : -1.0f;
    const float den = big ? w + fiy : (tiny ? y0 : w);
    const float q = div_fast(num, den);
    float res;
    if (big) {
        // (products with 2 are exact: fusing them changes no rounding)
        res = __builtin_fmaf(-2.0f, x - (q - r), fiy);
        if (__builtin_fabsf(x) < 0x1p-13f) res = fiy * __builtin_fmaf(-2.0f * fiy, x, 1.0f);
        res = u2f(f2u(res) ^ sgn);
    } else if (!odd) {
        res = tiny ? y0 : w;
    } else {
        // -1 / (x + r) to more than a float: the quotient and w cut to 12 bits, corrected by the products' remainders
        const float zc = u2f(f2u(w) & 0xfffff000u);
        const float vc = r - (zc - x);
        const float tc = u2f(f2u(q) & 0xfffff000u);
        const float sc = __builtin_fmaf(tc, zc, 1.0f);   // 12 x 12 bits: the product is exact
        res = tiny ? q : tc + q * (sc + tc * vc);
    }
    return res;
}

ZM_HD float sinf_glibc(float x, const SinCosCoef &k = SinCosCoef()) { return sincosf_glibc(x, 0, k); }
ZM_HD float cosf_glibc(float x, const SinCosCoef &k = SinCosCoef()) { return sincosf_glibc(x, 1, k); }

// atanf, asinf, acosf: fdlibm's s_atanf.c, e_asinf.c (the five-term polynomial glibc carries), e_acosf.c as
// glibc 2.35 ships them (these have no FMA build: the sources round every product).  The constants are
// the decimal literals of the sources; atanf returns pi/2 from |x| >= 2^25.  Equal to the host libm on
// all 2^32 inputs -- including the few Horner steps that are fused here because the exhaustive
// comparison shows no result changes, and, on the device, the short quotient and square root.
// Per argument range: numerator = n1 |x| + n0 and denominator = d1 |x| + d0 of the reduction, and
// atan of the range's centre as high + low part.  Ranges: |x| < 0.4375 (no reduction: |x| / 1),
// < 0.6875 ((2|x| - 1) / (2 + |x|)), < 1.1875 ((|x| - 1) / (|x| + 1)), < 2.4375 ((|x| - 1.5) / (1 + 1.5 |x|)),
// above (-1 / |x|).  Each n1 |x| + n0 as one fused multiply-add rounds like the sources' expression
// (the products are exact, except 1.5 |x|, where the exhaustive comparison shows no change).
#define ZM_ATANF_TAB                                                                                        \
    { 1.0f, 0.0f, 0.0f, 1.0f, 0.0f, 0.0f, 0.0f, 0.0f,                                                       \
      2.0f, -1.0f, 1.0f, 2.0f, 4.6364760399e-01f, 5.0121582440e-09f, 0.0f, 0.0f,                            \
      1.0f, -1.0f, 1.0f, 1.0f, 7.8539812565e-01f, 3.7748947079e-08f, 0.0f, 0.0f,                            \
      1.0f, -1.5f, 1.5f, 1.0f, 9.8279368877e-01f, 3.4473217170e-08f, 0.0f, 0.0f,                            \
      0.0f, -1.0f, 1.0f, 0.0f, 1.5707962513e+00f, 7.5497894159e-08f, 0.0f, 0.0f }
static const float kAtanfTabHost[40] = ZM_ATANF_TAB;
#if defined(__HIPCC__)
static __device__ const float kAtanfTabDev[40] = ZM_ATANF_TAB;
#endif
ZM_HD const float *atanf_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return kAtanfTabDev;
#else
    return kAtanfTabHost;
#endif
}

ZM_HD float atanf_fdlibm(float x, const float *tab)
{
    const float hi3 = 1.5707962513e+00f, lo3 = 7.5497894159e-08f;
    const float a0 = 3.3333334327e-01f, a1 = -2.0000000298e-01f, a2 = 1.4285714924e-01f, a3 = -1.1111110449e-01f,
                a4 = 9.0908870101e-02f, a5 = -7.6918758452e-02f, a6 = 6.6610731184e-02f, a7 = -5.8335702866e-02f,
                a8 = 4.9768779427e-02f, a9 = -3.6531571299e-02f, a10 = 1.6285819933e-02f;
    const uint32_t hx = f2u(x);
    const uint32_t ix = hx & 0x7fffffffu;
    if (__builtin_expect(ix >= 0x4c000000u, 0)) {        // |x| >= 2^25
        if (ix > 0x7f800000u) return x + x;              // NaN
        return (hx >> 31) ? -hi3 - lo3 : hi3 + lo3;
    }
    // One path for all five ranges (a wavefront holds arguments of several): the range picks a table
    // row, the reduced argument is one quotient, the sign goes back at the end (every step is odd
    // in x).  Without a reduction the sources return x - x (s1 + s2), which is h - ((x (s1 + s2) - l) - x)
    // with h = l = 0; below 2^-29 they return x, and so does this (s1 + s2 vanishes against 1).
    const uint32_t id = (uint32_t)(ix >= 0x3ee00000u) + (uint32_t)(ix >= 0x3f300000u) + (uint32_t)(ix >= 0x3f980000u) +
                        (uint32_t)(ix >= 0x401c0000u);
    const float *e = tab + 8 * id;
    const float ax = u2f(ix);
    const float num = __builtin_fmaf(e[0], ax, e[1]);
    const float den = __builtin_fmaf(e[2], ax, e[3]);
    const float h = e[4], l = e[5];
    const float xr = div_fast(num, den);
    const float z = xr * xr;
    const float w = z * z;
    // the inner Horner steps are fused where that changes none of the 2^32 results (each was tried
    // alone and together; fusing any of the others changes between 8 and 405 980 of them)
    float s1 = __builtin_fmaf(w, a10, a8);
    s1 = __builtin_fmaf(w, s1, a6);
    s1 = __builtin_fmaf(w, s1, a4);
    s1 = z * (a0 + w * (a2 + w * s1));
    float s2 = __builtin_fmaf(w, a9, a7);
    s2 = __builtin_fmaf(w, s2, a5);
    s2 = w * (a1 + w * (a3 + w * s2));
    const float r = h - ((xr * (s1 + s2) - l) - xr);
    return u2f(f2u(r) | (hx & 0x80000000u));
}
ZM_HD float atanf_fdlibm(float x) { return atanf_fdlibm(x, atanf_table()); }

ZM_HD float asinf_fdlibm(float x)
{
    const float one = 1.0f, pio2_hi = 1.57079637050628662109375f, pio2_lo = -4.37113900018624283e-8f,
                pio4_hi = 0.785398185253143310546875f;
    const float p0 = 1.666675248e-1f, p1 = 7.495297643e-2f, p2 = 4.547037598e-2f, p3 = 2.417951451e-2f,
                p4 = 4.216630880e-2f;
    const uint32_t hx = f2u(x);
    const uint32_t ix = hx & 0x7fffffffu;
    if (ix == 0x3f800000u) return x * pio2_hi + x * pio2_lo;     // asin(+-1) = +-pi/2
    // |x| > 1, NaN: the sources' (x - x) / (x - x); a NaN either way, without the division (a third of
    // normally distributed arguments end here, and a division is eleven instructions for the whole wavefront)
    if (ix > 0x3f800000u) return (x - x) * u2f(0x7f800000u);
    // both ranges evaluate the same polynomial, of x^2 below 0.5 and of (1 - |x|) / 2 above: once here
    const bool small = ix < 0x3f000000u;                 // |x| < 0.5
    if (small && ix < 0x32000000u) return x;             // |x| < 2^-27
    float w = one - u2f(ix);
    float t = small ? x * x : w * 0.5f;
    float p = t * (p0 + t * (p1 + t * (p2 + t * (p3 + t * p4))));
    if (small) return x + x * p;
    const float s = sqrt_fast(t);
    if (ix >= 0x3F79999Au) {                             // |x| > 0.975
        t = pio2_hi - (2.0f * (s + s * p) - pio2_lo);
    } else {
        w = u2f(f2u(s) & 0xfffff000u);
        const float c = div_fast(__builtin_fmaf(-w, w, t), s + w);   // w has 12 bits: w*w is exact
        const float r = p;
        p = 2.0f * s * r - (pio2_lo - 2.0f * c);
        const float q = pio4_hi - 2.0f * w;
        t = pio4_hi - (p - q);
    }
    return (hx >> 31) ? -t : t;
}

ZM_HD float acosf_fdlibm(float x)
{
    const float one = 1.0f, pi = 3.1415925026e+00f, pio2_hi = 1.5707962513e+00f, pio2_lo = 7.5497894159e-08f;
    const float pS0 = 1.6666667163e-01f, pS1 = -3.2556581497e-01f, pS2 = 2.0121252537e-01f, pS3 = -4.0055535734e-02f,
                pS4 = 7.9153501429e-04f, pS5 = 3.4793309169e-05f;
    const float qS1 = -2.4033949375e+00f, qS2 = 2.0209457874e+00f, qS3 = -6.8828397989e-01f, qS4 = 7.7038154006e-02f;
    const uint32_t hx = f2u(x);
    const uint32_t ix = hx & 0x7fffffffu;
    const bool neg = (hx >> 31) != 0;
    if (ix == 0x3f800000u) return neg ? pi + 2.0f * pio2_lo : 0.0f;   // acos(-1) = pi, acos(1) = 0
    if (ix > 0x3f800000u) return (x - x) * u2f(0x7f800000u);          // |x| > 1, NaN: the sources' (x - x) / (x - x) without the division
    // the three ranges evaluate the same rational function p(z) / q(z), of x^2, (1 + x) / 2 or
    // (1 - x) / 2: once here, whatever mix of ranges a wavefront holds
    const bool small = ix < 0x3f000000u;                 // |x| < 0.5
    if (small && ix <= 0x23000000u) return pio2_hi + pio2_lo;   // |x| < 2^-57
    const float z = small ? x * x : (neg ? (one + x) * 0.5f : (one - x) * 0.5f);
    // (the innermost step of p is the only one of the two polynomials that can be fused without
    // changing a result)
    const float p = z * (pS0 + z * (pS1 + z * (pS2 + z * (pS3 + z * __builtin_fmaf(z, pS5, pS4)))));
    const float q = one + z * (qS1 + z * (qS2 + z * (qS3 + z * qS4)));
    const float r = div_fast(p, q);
    if (small) return pio2_hi - (x - (pio2_lo - x * r));
    const float s = sqrt_fast(z);
    if (neg) {                                           // x < -0.5
        const float w = r * s - pio2_lo;
        return pi - 2.0f * (s + w);
    }
    const float df = u2f(f2u(s) & 0xfffff000u);          // x > 0.5
    const float c = div_fast(__builtin_fmaf(-df, df, z), s + df);   // df has 12 bits: df*df is exact
    const float w = r * s + c;
    return 2.0f * (df + w);
}

// ---- double precision exp: the table-driven routine glibc ships since 2.28 (from ARM's optimized routines) ----
// x = k ln2/N + r, N = 128;  exp(x) = 2^(k/N) exp(r),  2^(k/N) = H[k] (1 + tail[k]) with H the nearest
// double;  exp(r) - 1 as a degree-5 polynomial.  The table holds {tail[k], bits(H[k]) - (k << 52) / N};
// it is regenerated here from that definition with 80-digit arithmetic.  Fused multiply-adds as in
// the x86-64 build that CPUs with FMA select: every a + b*c of the main path, and the scale step of
// the overflow side of the special case, but not the underflow side (its product has two uses).
// Equal to the host libm's exp on 1.4e10 sampled inputs (uniform bit patterns, and uniform in
// +-745, +-30, +-1, +-2^-20), subnormal results included.
#define ZM_EXP_TAB                                                                                          \
    {                                                                                                       \
      0x0ull, 0x3ff0000000000000ull, 0x3c9b3b4f1a88bf6eull, 0x3feff63da9fb3335ull,                          \
      0xbc7160139cd8dc5dull, 0x3fefec9a3e778061ull, 0xbc905e7a108766d1ull, 0x3fefe315e86e7f85ull,           \
      0x3c8cd2523567f613ull, 0x3fefd9b0d3158574ull, 0xbc8bce8023f98efaull, 0x3fefd06b29ddf6deull,           \
      0x3c60f74e61e6c861ull, 0x3fefc74518759bc8ull, 0x3c90a3e45b33d399ull, 0x3fefbe3ecac6f383ull,           \
      0x3c979aa65d837b6dull, 0x3fefb5586cf9890full, 0x3c8eb51a92fdeffcull, 0x3fefac922b7247f7ull,           \
      0x3c3ebe3d702f9cd1ull, 0x3fefa3ec32d3d1a2ull, 0xbc6a033489906e0bull, 0x3fef9b66affed31bull,           \
      0xbc9556522a2fbd0eull, 0x3fef9301d0125b51ull, 0xbc5080ef8c4eea55ull, 0x3fef8abdc06c31ccull,           \
      0xbc91c923b9d5f416ull, 0x3fef829aaea92de0ull, 0x3c80d3e3e95c55afull, 0x3fef7a98c8a58e51ull,           \
      0xbc801b15eaa59348ull, 0x3fef72b83c7d517bull, 0xbc8f1ff055de323dull, 0x3fef6af9388c8deaull,           \
      0x3c8b898c3f1353bfull, 0x3fef635beb6fcb75ull, 0xbc96d99c7611eb26ull, 0x3fef5be084045cd4ull,           \
      0x3c9aecf73e3a2f60ull, 0x3fef54873168b9aaull, 0xbc8fe782cb86389dull, 0x3fef4d5022fcd91dull,           \
      0x3c8a6f4144a6c38dull, 0x3fef463b88628cd6ull, 0x3c807a05b0e4047dull, 0x3fef3f49917ddc96ull,           \
      0x3c968efde3a8a894ull, 0x3fef387a6e756238ull, 0x3c875e18f274487dull, 0x3fef31ce4fb2a63full,           \
      0x3c80472b981fe7f2ull, 0x3fef2b4565e27cddull, 0xbc96b87b3f71085eull, 0x3fef24dfe1f56381ull,           \
      0x3c82f7e16d09ab31ull, 0x3fef1e9df51fdee1ull, 0xbc3d219b1a6fbffaull, 0x3fef187fd0dad990ull,           \
      0x3c8b3782720c0ab4ull, 0x3fef1285a6e4030bull, 0x3c6e149289cecb8full, 0x3fef0cafa93e2f56ull,           \
      0x3c834d754db0abb6ull, 0x3fef06fe0a31b715ull, 0x3c864201e2ac744cull, 0x3fef0170fc4cd831ull,           \
      0x3c8fdd395dd3f84aull, 0x3feefc08b26416ffull, 0xbc86a3803b8e5b04ull, 0x3feef6c55f929ff1ull,           \
      0xbc924aedcc4b5068ull, 0x3feef1a7373aa9cbull, 0xbc9907f81b512d8eull, 0x3feeecae6d05d866ull,           \
      0xbc71d1e83e9436d2ull, 0x3feee7db34e59ff7ull, 0xbc991919b3ce1b15ull, 0x3feee32dc313a8e5ull,           \
      0x3c859f48a72a4c6dull, 0x3feedea64c123422ull, 0xbc9312607a28698aull, 0x3feeda4504ac801cull,           \
      0xbc58a78f4817895bull, 0x3feed60a21f72e2aull, 0xbc7c2c9b67499a1bull, 0x3feed1f5d950a897ull,           \
      0x3c4363ed60c2ac11ull, 0x3feece086061892dull, 0x3c9666093b0664efull, 0x3feeca41ed1d0057ull,           \
      0x3c6ecce1daa10379ull, 0x3feec6a2b5c13cd0ull, 0x3c93ff8e3f0f1230ull, 0x3feec32af0d7d3deull,           \
      0x3c7690cebb7aafb0ull, 0x3feebfdad5362a27ull, 0x3c931dbdeb54e077ull, 0x3feebcb299fddd0dull,           \
      0xbc8f94340071a38eull, 0x3feeb9b2769d2ca7ull, 0xbc87deccdc93a349ull, 0x3feeb6daa2cf6642ull,           \
      0xbc78dec6bd0f385full, 0x3feeb42b569d4f82ull, 0xbc861246ec7b5cf6ull, 0x3feeb1a4ca5d920full,           \
      0x3c93350518fdd78eull, 0x3feeaf4736b527daull, 0x3c7b98b72f8a9b05ull, 0x3feead12d497c7fdull,           \
      0x3c9063e1e21c5409ull, 0x3feeab07dd485429ull, 0x3c34c7855019c6eaull, 0x3feea9268a5946b7ull,           \
      0x3c9432e62b64c035ull, 0x3feea76f15ad2148ull, 0xbc8ce44a6199769full, 0x3feea5e1b976dc09ull,           \
      0xbc8c33c53bef4da8ull, 0x3feea47eb03a5585ull, 0xbc845378892be9aeull, 0x3feea34634ccc320ull,           \
      0xbc93cedd78565858ull, 0x3feea23882552225ull, 0x3c5710aa807e1964ull, 0x3feea155d44ca973ull,           \
      0xbc93b3efbf5e2228ull, 0x3feea09e667f3bcdull, 0xbc6a12ad8734b982ull, 0x3feea012750bdabfull,           \
      0xbc6367efb86da9eeull, 0x3fee9fb23c651a2full, 0xbc80dc3d54e08851ull, 0x3fee9f7df9519484ull,           \
      0xbc781f647e5a3ecfull, 0x3fee9f75e8ec5f74ull, 0xbc86ee4ac08b7db0ull, 0x3fee9f9a48a58174ull,           \
      0xbc8619321e55e68aull, 0x3fee9feb564267c9ull, 0x3c909ccb5e09d4d3ull, 0x3feea0694fde5d3full,           \
      0xbc7b32dcb94da51dull, 0x3feea11473eb0187ull, 0x3c94ecfd5467c06bull, 0x3feea1ed0130c132ull,           \
      0x3c65ebe1abd66c55ull, 0x3feea2f336cf4e62ull, 0xbc88a1c52fb3cf42ull, 0x3feea427543e1a12ull,           \
      0xbc9369b6f13b3734ull, 0x3feea589994cce13ull, 0xbc805e843a19ff1eull, 0x3feea71a4623c7adull,           \
      0xbc94d450d872576eull, 0x3feea8d99b4492edull, 0x3c90ad675b0e8a00ull, 0x3feeaac7d98a6699ull,           \
      0x3c8db72fc1f0eab4ull, 0x3feeace5422aa0dbull, 0xbc65b6609cc5e7ffull, 0x3feeaf3216b5448cull,           \
      0x3c7bf68359f35f44ull, 0x3feeb1ae99157736ull, 0xbc93091fa71e3d83ull, 0x3feeb45b0b91ffc6ull,           \
      0xbc5da9b88b6c1e29ull, 0x3feeb737b0cdc5e5ull, 0xbc6c23f97c90b959ull, 0x3feeba44cbc8520full,           \
      0xbc92434322f4f9aaull, 0x3feebd829fde4e50ull, 0xbc85ca6cd7668e4bull, 0x3feec0f170ca07baull,           \
      0x3c71affc2b91ce27ull, 0x3feec49182a3f090ull, 0x3c6dd235e10a73bbull, 0x3feec86319e32323ull,           \
      0xbc87c50422622263ull, 0x3feecc667b5de565ull, 0x3c8b1c86e3e231d5ull, 0x3feed09bec4a2d33ull,           \
      0xbc91bbd1d3bcbb15ull, 0x3feed503b23e255dull, 0x3c90cc319cee31d2ull, 0x3feed99e1330b358ull,           \
      0x3c8469846e735ab3ull, 0x3feede6b5579fdbfull, 0xbc82dfcd978e9db4ull, 0x3feee36bbfd3f37aull,           \
      0x3c8c1a7792cb3387ull, 0x3feee89f995ad3adull, 0xbc907b8f4ad1d9faull, 0x3feeee07298db666ull,           \
      0xbc55c3d956dcaebaull, 0x3feef3a2b84f15fbull, 0xbc90a40e3da6f640ull, 0x3feef9728de5593aull,           \
      0xbc68d6f438ad9334ull, 0x3feeff76f2fb5e47ull, 0xbc91eee26b588a35ull, 0x3fef05b030a1064aull,           \
      0x3c74ffd70a5fddcdull, 0x3fef0c1e904bc1d2ull, 0xbc91bdfbfa9298acull, 0x3fef12c25bd71e09ull,           \
      0x3c736eae30af0cb3ull, 0x3fef199bdd85529cull, 0x3c8ee3325c9ffd94ull, 0x3fef20ab5fffd07aull,           \
      0x3c84e08fd10959acull, 0x3fef27f12e57d14bull, 0x3c63cdaf384e1a67ull, 0x3fef2f6d9406e7b5ull,           \
      0x3c676b2c6c921968ull, 0x3fef3720dcef9069ull, 0xbc808a1883ccb5d2ull, 0x3fef3f0b555dc3faull,           \
      0xbc8fad5d3ffffa6full, 0x3fef472d4a07897cull, 0xbc900dae3875a949ull, 0x3fef4f87080d89f2ull,           \
      0x3c74a385a63d07a7ull, 0x3fef5818dcfba487ull, 0xbc82919e2040220full, 0x3fef60e316c98398ull,           \
      0x3c8e5a50d5c192acull, 0x3fef69e603db3285ull, 0x3c843a59ac016b4bull, 0x3fef7321f301b460ull,           \
      0xbc82d52107b43e1full, 0x3fef7c97337b9b5full, 0xbc892ab93b470dc9ull, 0x3fef864614f5a129ull,           \
      0x3c74b604603a88d3ull, 0x3fef902ee78b3ff6ull, 0x3c83c5ec519d7271ull, 0x3fef9a51fbc74c83ull,           \
      0xbc8ff7128fd391f0ull, 0x3fefa4afa2a490daull, 0xbc8dae98e223747dull, 0x3fefaf482d8e67f1ull,           \
      0x3c8ec3bc41aa2008ull, 0x3fefba1bee615a27ull, 0x3c842b94c3a9eb32ull, 0x3fefc52b376bba97ull,           \
      0x3c8a64a931d185eeull, 0x3fefd0765b6e4540ull, 0xbc8e37bae43be3edull, 0x3fefdbfdad9cbe14ull,           \
      0x3c77893b4d91cd9dull, 0x3fefe7c1819e90d8ull, 0x3c5305c14160cc89ull, 0x3feff3c22b8f71f1ull }

static const uint64_t kExpTabHost[256] = ZM_EXP_TAB;
#if defined(__HIPCC__)
static __device__ const uint64_t kExpTabDev[256] = ZM_EXP_TAB;
#endif
ZM_HD const uint64_t *exp_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return kExpTabDev;
#else
    return kExpTabHost;
#endif
}

// The constants of the f64 routines as data: handed to a kernel as part of its argument they sit in
// scalar registers and feed the f64 operations directly; written as literals each one is moved into
// a register pair before every use, two scalar instructions per constant and element, and the one
// scalar unit of a CU serves all four SIMDs.
struct ExpCoef64 {
    double inv_ln2n = 0x1.71547652b82fep0 * 128, neg_ln2hi_n = -0x1.62e42fefa0000p-8, neg_ln2lo_n = -0x1.cf79abc9e3b3ap-47,
           shift = 0x1.8p52;
    double c2 = 0x1.ffffffffffdbdp-2, c3 = 0x1.555555555543cp-3, c4 = 0x1.55555cf172b91p-5, c5 = 0x1.1111167a4d017p-7;
};
struct Expm1Coef64 {   // fdlibm's expm1: ln2 in two parts, 1/ln2, Q1..Q5
    double ln2_hi = 0x1.62e42feep-1, ln2_lo = 0x1.a39ef35793c76p-33, invln2 = 0x1.71547652b82fep+0;
    double q1 = -0x1.11111111110f4p-5, q2 = 0x1.a01a019fe5585p-10, q3 = -0x1.4ce199eaadbb7p-14, q4 = 0x1.0cfca86e65239p-18,
           q5 = -0x1.afdb76e09c32dp-23;
};

ZM_HD double exp_glibc(double x, const uint64_t *tab, const ExpCoef64 &k = ExpCoef64())
{
    const double InvLn2N = k.inv_ln2n, NegLn2hiN = k.neg_ln2hi_n, NegLn2loN = k.neg_ln2lo_n, Shift = k.shift;
    const double C2 = k.c2, C3 = k.c3, C4 = k.c4, C5 = k.c5;
    uint32_t abstop = (uint32_t)(d2u(x) >> 52) & 0x7ffu;
    if (abstop - 0x3c9u >= 0x408u - 0x3c9u) {            // |x| < 2^-54, |x| >= 512, inf or NaN
        if (abstop - 0x3c9u >= 0x80000000u) return 1.0 + x;
        if (abstop >= 0x409u) {                          // |x| >= 1024
            if (d2u(x) == 0xfff0000000000000ull) return 0.0;
            if (abstop >= 0x7ffu) return 1.0 + x;
            return (d2u(x) >> 63) ? 0.0 : u2d(0x7ff0000000000000ull);
        }
        abstop = 0;                                      // large |x|: the special case below
    }
    const double z = InvLn2N * x;
    double kd = z + Shift;
    const uint64_t ki = d2u(kd);
    kd -= Shift;
    const double r = __builtin_fma(kd, NegLn2loN, __builtin_fma(kd, NegLn2hiN, x));
    const uint64_t idx = 2 * (ki % 128);
    const uint64_t top = ki << (52 - 7);
    const double tail = u2d(tab[idx]);
    uint64_t sbits = tab[idx + 1] + top;
    const double r2 = r * r;
    const double tmp = __builtin_fma(r2 * r2, __builtin_fma(r, C5, C4), __builtin_fma(r2, __builtin_fma(r, C3, C2), tail + r));
    if (abstop == 0) {
        if ((ki & 0x80000000u) == 0) {                   // k > 0: the exponent of scale may have overflowed
            sbits -= 1009ull << 52;
            const double scale = u2d(sbits);
            return 0x1p1009 * __builtin_fma(scale, tmp, scale);
        }
        sbits += 1022ull << 52;                          // k < 0: care in the subnormal range
        const double scale = u2d(sbits);
        double y = scale + scale * tmp;
        if (y < 1.0) {
            double lo = scale - y + scale * tmp;
            const double hi = 1.0 + y;
            lo = 1.0 - hi + y + lo;
            y = (hi + lo) - 1.0;
            if (y == 0.0) y = 0.0;
        }
        return 0x1p-1022 * y;
    }
    const double scale = u2d(sbits);
    return __builtin_fma(scale, tmp, scale);
}
ZM_HD double exp_glibc(double x) { return exp_glibc(x, exp_table()); }
// the main path alone, for callers whose argument needs none of the special cases (2^-54 <= |x| < 512)
ZM_HD double exp_glibc_core(double x, const uint64_t *tab, const ExpCoef64 &k = ExpCoef64())
{
    const double z = k.inv_ln2n * x;
    double kd = z + k.shift;
    const uint64_t ki = d2u(kd);
    kd -= k.shift;
    const double r = __builtin_fma(kd, k.neg_ln2lo_n, __builtin_fma(kd, k.neg_ln2hi_n, x));
    const uint64_t idx = 2 * (ki % 128);
    const uint64_t top = ki << (52 - 7);
    const double tail = u2d(tab[idx]);
    const uint64_t sbits = tab[idx + 1] + top;
    const double r2 = r * r;
    const double tmp = __builtin_fma(r2 * r2, __builtin_fma(r, k.c5, k.c4), __builtin_fma(r2, __builtin_fma(r, k.c3, k.c2), tail + r));
    const double scale = u2d(sbits);
    return __builtin_fma(scale, tmp, scale);
}

// ---- double precision: fdlibm s_expm1.c / s_tanh.c as shipped by glibc 2.35 (generic dbl-64) ----------

ZM_HD uint64_t d2u(double d)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return (uint64_t)__double_as_longlong(d);
#else
    uint64_t u;
    memcpy(&u, &d, 8);
    return u;
#endif
}
ZM_HD double u2d(uint64_t u)
{
#if defined(__HIP_DEVICE_COMPILE__)
    return __longlong_as_double((long long)u);
#else
    double d;
    memcpy(&d, &u, 8);
    return d;
#endif
}
ZM_HD uint32_t hi_word(double d) { return (uint32_t)(d2u(d) >> 32); }
ZM_HD double add_to_hi_word(double d, uint32_t inc) { return u2d(d2u(d) + ((uint64_t)inc << 32)); }
ZM_HD double from_hi_word(uint32_t hi) { return u2d((uint64_t)hi << 32); }

// expm1 for finite arguments (tanh passes |x| < 44)
ZM_HD double expm1_fdlibm(double x)
{
    const double one = 1.0, tiny = 1.0e-300, huge = 1.0e+300;
    const double o_threshold = 7.09782712893383973096e+02;
    const double ln2_hi = u2d(0x3fe62e42fee00000ull);   // 6.93147180369123816490e-01
    const double ln2_lo = u2d(0x3dea39ef35793c76ull);   // 1.90821492927058770002e-10
    const double invln2 = u2d(0x3ff71547652b82feull);   // 1.44269504088896338700e+00
    const double Q1 = u2d(0xBFA11111111110F4ull);       // -3.33333333333331316428e-02
    const double Q2 = u2d(0x3F5A01A019FE5585ull);       //  1.58730158725481460165e-03
    const double Q3 = u2d(0xBF14CE199EAADBB7ull);       // -7.93650757867487942473e-05
    const double Q4 = u2d(0x3ED0CFCA86E65239ull);       //  4.00821782732936239552e-06
    const double Q5 = u2d(0xBE8AFDB76E09C32Dull);       // -2.01099218183624371326e-07

    double y, hi, lo, c = 0.0, t, e, hxs, hfx, r1, h2, h4, R1, R2, R3;
    int32_t k;
    uint32_t hx = hi_word(x);
    const uint32_t xsb = hx & 0x80000000u;
    hx &= 0x7fffffffu;

    if (hx >= 0x4043687Au) {                 // |x| >= 56 ln2
        if (hx >= 0x40862E42u) {             // |x| >= 709.78...
            if (hx >= 0x7ff00000u) {
                if (((hx & 0xfffffu) | (uint32_t)d2u(x)) != 0) return x + x;   // NaN
                return (xsb == 0) ? x : -1.0;                                 // +-inf
            }
            if (x > o_threshold) return huge * huge;
        }
        if (xsb != 0) return tiny - one;     // x < -56 ln2
    }
    if (hx > 0x3fd62e42u) {                  // |x| > 0.5 ln2
        if (hx < 0x3FF0A2B2u) {              // |x| < 1.5 ln2
            if (xsb == 0) { hi = x - ln2_hi; lo = ln2_lo;  k = 1; }
            else          { hi = x + ln2_hi; lo = -ln2_lo; k = -1; }
        } else {
            k = (int32_t)(invln2 * x + ((xsb == 0) ? 0.5 : -0.5));
            t = (double)k;
            hi = x - t * ln2_hi;
            lo = t * ln2_lo;
        }
        x = hi - lo;
        c = (hi - x) - lo;
    } else if (hx < 0x3c900000u) {           // |x| < 2^-54
        t = huge + x;
        return x - (t - (huge + x));
    } else {
        k = 0;
    }
    hfx = 0.5 * x;
    hxs = x * hfx;
    R1 = one + hxs * Q1;
    h2 = hxs * hxs;
    R2 = Q2 + hxs * Q3;
    h4 = h2 * h2;
    R3 = Q4 + hxs * Q5;
    r1 = R1 + h2 * R2 + h4 * R3;
    t = 3.0 - r1 * hfx;
    e = hxs * ((r1 - t) / (6.0 - x * t));
    if (k == 0) return x - (x * e - hxs);
    e = (x * (e - c) - c);
    e -= hxs;
    if (k == -1) return 0.5 * (x - e) - 0.5;
    if (k == 1) {
        if (x < -0.25) return -2.0 * (e - (x + 0.5));
        return one + 2.0 * (x - e);
    }
    if (k <= -2 || k > 56) {
        y = one - (e - x);
        y = add_to_hi_word(y, (uint32_t)k << 20);
        return y - one;
    }
    if (k < 20) {
        t = from_hi_word(0x3ff00000u - (0x200000u >> k));   // 1 - 2^-k
        y = t - (e - x);
        y = add_to_hi_word(y, (uint32_t)k << 20);
    } else {
        t = from_hi_word((uint32_t)(0x3ff - k) << 20);      // 2^-k
        y = x - (e + t);
        y += one;
        y = add_to_hi_word(y, (uint32_t)k << 20);
    }
    return y;
}

ZM_HD double tanh_fdlibm(double x)
{
    const double one = 1.0, two = 2.0, tiny = 1.0e-300;
    const uint64_t bits = d2u(x);
    const uint32_t jx = (uint32_t)(bits >> 32), lx = (uint32_t)bits;
    const uint32_t ix = jx & 0x7fffffffu;
    const bool neg = (jx >> 31) != 0;
    double t, z;
    if (ix >= 0x7ff00000u) return neg ? one / x - one : one / x + one;   // inf or NaN
    if (ix < 0x40360000u) {                  // |x| < 22
        if ((ix | lx) == 0) return x;        // +-0
        if (ix < 0x3c800000u) return x * (one + x);   // |x| < 2^-55
        const double ax = u2d(bits & 0x7fffffffffffffffull);
        if (ix >= 0x3ff00000u) {             // |x| >= 1
            t = expm1_fdlibm(two * ax);
            z = one - two / (t + two);
        } else {
            t = expm1_fdlibm(-two * ax);
            z = -t / (t + two);
        }
    } else {
        z = one - tiny;
    }
    return neg ? -z : z;
}

// The same tanh for 64-wide execution, as tanhf_simd_core does it in f32, but with only those
// rewrites that perform fdlibm's operations on fdlibm's operands (no f64 function can be compared on
// all of its arguments, so nothing here rests on an exhaustive check):
//   * one path through the argument reduction, the rational core and one division pair; k is fdlibm's
//     (0 up to 0.5 ln2 by the high word, trunc(a/ln2 +- 0.5) above; between 0.5 ln2 and 1.5 ln2 the
//     sources take k = +-1 with hi = a -+ ln2_hi, lo = +-ln2_lo, which is what the general formula gives:
//     the bounds on the high word keep a/ln2 +- 0.5 inside (1, 2));
//   * hi = a - k ln2_hi fused: ln2_hi ends in 21 zero bits, the product is exact;
//   * |a| < 2^-54 (expm1 returns a) and |x| < 2^-55 (tanh returns x (1 + x) = x) go through the k = 0
//     formula, whose correction term is below half a unit in the last place there;
//   * the tails share d = e1 - xr: k = 0 is -d (c is 0 there), k = -1 is -0.5 d - 0.5 in one fused step
//     (exact product), k <= -2 and 3 <= k < 20 are (A - d) 2^k with A = 1 (and a final - 1) or
//     A = 1 - 2^-k, whose bit pattern comes out as 1 for the negative k; |x| >= 1 decides which;
//   * |x| >= 6.5 (k could reach 20), infinities and NaN go to tanh_fdlibm.
// The core works on a2 = 2|x|; the sigmoid passes |x| (see sigmoidf_zenu).
ZM_HD double tanh_simd_core(double a2, double x, const Expm1Coef64 &ck = Expm1Coef64())
{
    const double one = 1.0, two = 2.0;
    const double ln2_hi = ck.ln2_hi, ln2_lo = ck.ln2_lo, invln2 = ck.invln2;
    const double Q1 = ck.q1, Q2 = ck.q2, Q3 = ck.q3, Q4 = ck.q4, Q5 = ck.q5;
    const bool big = a2 >= two;              // |x| >= 1: expm1(+2|x|), else expm1(-2|x|)
    const double a = big ? a2 : -a2;
    int32_t k = (int32_t)(invln2 * a + (big ? 0.5 : -0.5));
    k = (hi_word(a2) > 0x3fd62e42u) ? k : 0;
    const double tk = (double)k;
    const double hi = __builtin_fma(-tk, ln2_hi, a);
    const double lo = tk * ln2_lo;
    const double xr = hi - lo;
    const double c = (hi - xr) - lo;
    const double hfx = 0.5 * xr;
    const double hxs = xr * hfx;
    const double R1 = one + hxs * Q1;
    const double h2 = hxs * hxs;
    const double R2 = Q2 + hxs * Q3;
    const double h4 = h2 * h2;
    const double R3 = Q4 + hxs * Q5;
    const double r1 = R1 + h2 * R2 + h4 * R3;
    const double t = 3.0 - r1 * hfx;
    const double e = hxs * ((r1 - t) / (6.0 - xr * t));
    double e1 = xr * (e - c) - c;
    e1 -= hxs;
    const double d = e1 - xr;
    const double mneg1 = __builtin_fma(-0.5, d, -0.5);
    const double tt = from_hi_word(0x3ff00000u - (0x200000u >> (k & 31)));
    const double y = tt - d;
    const double ys = add_to_hi_word(y, (uint32_t)k << 20);
    double em1 = big ? ys : ys - one;
    em1 = (k == -1) ? mneg1 : em1;
    em1 = (k == 0) ? -d : em1;
    const double q = (big ? two : em1) / (em1 + two);
    const double z = big ? one - q : -q;
    return u2d((d2u(z) & 0x7fffffffffffffffull) | (d2u(x) & 0x8000000000000000ull));
}

ZM_RARE double tanh_rare(double x) { return tanh_fdlibm(x); }

ZM_HD double tanh_simd(double x, const Expm1Coef64 &ck = Expm1Coef64())
{
    const double ax = u2d(d2u(x) & 0x7fffffffffffffffull);
    if (__builtin_expect(!(ax < 6.5), 0)) return tanh_rare(x);
    return tanh_simd_core(ax + ax, x, ck);
}

// ZeNu's sigmoid composite in f64: tanh(x/2) needs 2|x/2| = |x| (where x/2 underflows and rounds,
// tanh is below 2^-1022 either way and vanishes against 0.5); 0.5 tanh is exact or vanishes, so
// the last two steps are one fused multiply-add
ZM_HD double sigmoid_zenu(double x, const Expm1Coef64 &ck = Expm1Coef64())
{
    const double ax = u2d(d2u(x) & 0x7fffffffffffffffull);
    if (__builtin_expect(!(ax < 13.0), 0)) {
        const double th = tanh_rare(x * 0.5);
        return 0.5 + 0.5 * th;
    }
    return __builtin_fma(0.5, tanh_simd_core(ax, x, ck), 0.5);
}

// sinh / cosh in f64 (fdlibm e_sinh.c / e_cosh.c as glibc 2.35 ships them) over the expm1 and exp above
ZM_HD double sinh_fdlibm(double x, const uint64_t *etab)
{
    const double one = 1.0, shuge = 1.0e307;
    const uint32_t jx = hi_word(x);
    const uint32_t ix = jx & 0x7fffffffu;
    if (ix >= 0x7ff00000u) return x + x;                 // inf, NaN
    const double h = (jx & 0x80000000u) ? -0.5 : 0.5;
    const double ax = u2d(d2u(x) & 0x7fffffffffffffffull);
    if (ix < 0x40360000u) {                              // |x| < 22
        if (ix < 0x3e300000u) return x;                  // |x| < 2^-28
        const double t = expm1_fdlibm(ax);
        if (ix < 0x3ff00000u) return h * (2.0 * t - t * t / (t + one));
        return h * (t + t / (t + one));
    }
    if (ix < 0x40862e42u) return h * exp_glibc(ax, etab);    // |x| < log(DBL_MAX)
    const uint32_t lx = (uint32_t)d2u(x);
    if (ix < 0x408633ceu || (ix == 0x408633ceu && lx <= 0x8fb9f87du)) {
        const double w = exp_glibc(0.5 * ax, etab);
        const double t = h * w;
        return t * w;
    }
    return x * shuge;                                    // overflow
}

// sinh in f64 for 64-wide execution, with the means of tanh_simd_core (only rewrites that keep
// fdlibm's operations and operands): expm1(|x|) on one path with the tails k = 0, k = 1 in both of
// its forms and 2 <= k < 20 side by side, one division for both of sinh's ranges.  |x| >= 13
// (k could reach 20), infinities and NaN go to sinh_fdlibm; |x| < 2^-28 returns x as in the sources.
ZM_RARE double sinh_rare(double x, const uint64_t *etab) { return sinh_fdlibm(x, etab); }

ZM_HD double sinh_simd(double x, const uint64_t *etab, const Expm1Coef64 &ck = Expm1Coef64())
{
    const double one = 1.0;
    const double ln2_hi = ck.ln2_hi, ln2_lo = ck.ln2_lo, invln2 = ck.invln2;
    const double Q1 = ck.q1, Q2 = ck.q2, Q3 = ck.q3, Q4 = ck.q4, Q5 = ck.q5;
    const double a = u2d(d2u(x) & 0x7fffffffffffffffull);
    if (__builtin_expect(!(a < 13.0), 0)) return sinh_rare(x, etab);
    const uint32_t ix = hi_word(a);
    int32_t k = (int32_t)(invln2 * a + 0.5);
    k = (ix > 0x3fd62e42u) ? k : 0;
    const double tk = (double)k;
    const double hi = __builtin_fma(-tk, ln2_hi, a);     // the product is exact
    const double lo = tk * ln2_lo;
    const double xr = hi - lo;
    const double c = (hi - xr) - lo;
    const double hfx = 0.5 * xr;
    const double hxs = xr * hfx;
    const double R1 = one + hxs * Q1;
    const double h2 = hxs * hxs;
    const double R2 = Q2 + hxs * Q3;
    const double h4 = h2 * h2;
    const double R3 = Q4 + hxs * Q5;
    const double r1 = R1 + h2 * R2 + h4 * R3;
    const double t = 3.0 - r1 * hfx;
    const double e = hxs * ((r1 - t) / (6.0 - xr * t));
    double e1 = xr * (e - c) - c;
    e1 -= hxs;
    const double d = e1 - xr;
    const double k1b = __builtin_fma(-2.0, d, one);      // 1 + 2 (xr - e1): the doubling is exact
    const double k1a = -2.0 * (e1 - (xr + 0.5));
    const double k1 = (xr < -0.25) ? k1a : k1b;
    const double tt = from_hi_word(0x3ff00000u - (0x200000u >> (k & 31)));
    const double y = tt - d;
    double em1 = add_to_hi_word(y, (uint32_t)k << 20);
    em1 = (k == 1) ? k1 : em1;
    em1 = (k == 0) ? -d : em1;                           // c is 0: xr - (xr e - hxs) = -d
    const bool small = a < one;
    const double q = (small ? em1 * em1 : em1) / (em1 + one);
    const double r = small ? __builtin_fma(2.0, em1, -q) : em1 + q;   // 2 em1 is exact
    const double res = u2d(d2u(0.5 * r) | (d2u(x) & 0x8000000000000000ull));
    return (ix < 0x3e300000u) ? x : res;
}

ZM_HD double cosh_fdlibm(double x, const uint64_t *etab)
{
    const double one = 1.0, half = 0.5, huge = 1.0e300;
    const uint32_t ix = hi_word(x) & 0x7fffffffu;
    const double ax = u2d(d2u(x) & 0x7fffffffffffffffull);
    if (ix < 0x40360000u) {                              // |x| < 22
        if (ix < 0x3fd62e43u) {                          // |x| < 0.5 ln2
            if (ix < 0x3c800000u) return one;
            const double t = expm1_fdlibm(ax);
            const double w = one + t;
            return one + (t * t) / (w + w);
        }
        const double t = exp_glibc(ax, etab);
        return half * t + half / t;
    }
    if (ix < 0x40862e42u) return half * exp_glibc(ax, etab);
    const uint32_t lx = (uint32_t)d2u(x);
    if (ix < 0x408633ceu || (ix == 0x408633ceu && lx <= 0x8fb9f87du)) {
        const double w = exp_glibc(half * ax, etab);
        const double t = half * w;
        return t * w;
    }
    if (ix >= 0x7ff00000u) return x * x;                 // inf, NaN
    return huge * huge;                                  // overflow
}
// cosh in f64 as the kernels call it: below 0.5 ln2 expm1's k = 0 path written out (the general
// expm1 brings all of its branches along; below 2^-54, where it returns its argument, and below 2^-55,
// where cosh returns 1, the k = 0 formula gives the same), exp above, |x| >= 22 out of line.
ZM_RARE double cosh_rare(double x, const uint64_t *etab) { return cosh_fdlibm(x, etab); }
ZM_HD double cosh_simd(double x, const uint64_t *etab, const Expm1Coef64 &ck = Expm1Coef64(), const ExpCoef64 &ek = ExpCoef64())
{
    const double one = 1.0, half = 0.5;
    const double a = u2d(d2u(x) & 0x7fffffffffffffffull);
    if (__builtin_expect(!(a < 22.0), 0)) return cosh_rare(x, etab);
    if (hi_word(a) < 0x3fd62e43u) {                      // |x| < 0.5 ln2
        const double Q1 = ck.q1, Q2 = ck.q2, Q3 = ck.q3, Q4 = ck.q4, Q5 = ck.q5;
        const double hfx = half * a;
        const double hxs = a * hfx;
        const double R1 = one + hxs * Q1;
        const double h2 = hxs * hxs;
        const double R2 = Q2 + hxs * Q3;
        const double h4 = h2 * h2;
        const double R3 = Q4 + hxs * Q5;
        const double r1 = R1 + h2 * R2 + h4 * R3;
        const double t3 = 3.0 - r1 * hfx;
        const double e = hxs * ((r1 - t3) / (6.0 - a * t3));
        const double t = a - (a * e - hxs);
        const double w = one + t;
        return one + (t * t) / (w + w);
    }
    const double t = exp_glibc_core(a, etab, ek);        // 0.34 <= a < 22: none of exp's special cases
    return half * t + half / t;
}

ZM_HD double sinh_fdlibm(double x) { return sinh_fdlibm(x, exp_table()); }
ZM_HD double cosh_fdlibm(double x) { return cosh_fdlibm(x, exp_table()); }

// ZeNu's sigmoid composite in f32: each step rounded to f32, as the four autograd ops do.
ZM_HD float sigmoidf_zenu(float x, const TanhRegs &rg = TanhRegs())
{
    const float half = 0.5f;
    // tanh(x/2) needs 2|x/2| = |x|.  (Where x/2 underflows and rounds, tanh is below 2^-126 either
    // way and vanishes against 0.5.)
    float th = tanhf_simd_core(u2f(f2u(x) & 0x7fffffffu), x, rg);
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_fmaf(half, th, half);   // half*th is exact or vanishes against 0.5: same bits
#else
    float ht = half * th;
    return half + ht;
#endif
}

// tanh of an f32 evaluated in f64 and rounded once: NOT the host library's bits, but never more
// than 2 units in the last place away from them (the largest distance over all 2^32 arguments
// is 2: 97.23 % equal, 2.76 % one apart, 0.017 % two apart) in about 37 vector instructions.
// (tanhf_simd has since come down to 57 and is the faster of the two: its f32 instructions cost one
// issue slot each, the f64 division and conversions here more.)  tanh|x| = em1 / (em1 + 2) with em1 = exp(2|x|) - 1 = 2^k (1 + r p(r)) - 1, where
// 2|x| = k ln2 + r, |r| <= ln2 / 2, and p is a degree-8 fit of (exp(r) - 1) / r (relative error
// of exp below 2^-44).  With k = 0 the term 2^k - 1 vanishes and em1 = r p(r) keeps its relative
// accuracy down to the smallest subnormal.  Only IEEE operations, so host and device agree bit
// for bit.
// The constants travel as data (a kernel argument, so they sit in scalar registers and feed the
// f64 fused multiply-adds directly; written as literals the compiler copies each one into a pair
// of vector registers per use, a quarter of all instructions).
struct TanhUlp2Coef {
    double log2e = 1.4426950408889634;
    double ln2_hi = 6.93147180369123816490e-01, ln2_lo = 1.90821492927058770002e-10;
    double c[8] = {4.99999999997978561e-01, 1.66666666666491048e-01, 4.16666668910626939e-02,
                   8.33333335336592686e-03, 1.38888216534793383e-03, 1.98412091860510867e-04,
                   2.48761782309482669e-05, 2.76249453147040650e-06};   // c[i] multiplies r^(i+1); c0 = 1
};

ZM_HD float tanhf_ulp2(float x, const TanhUlp2Coef &q)
{
    float af = fabsf(x);
    af = af > 20.0f ? 20.0f : af;        // beyond 20 the quotient rounds to 1; a NaN stays a NaN
    const double a2 = 2.0 * (double)af;
    const double kd = rint(a2 * q.log2e);
    double r = fma(-kd, q.ln2_hi, a2);
    r = fma(-kd, q.ln2_lo, r);
    double p = q.c[7];
    p = fma(p, r, q.c[6]);
    p = fma(p, r, q.c[5]);
    p = fma(p, r, q.c[4]);
    p = fma(p, r, q.c[3]);
    p = fma(p, r, q.c[2]);
    p = fma(p, r, q.c[1]);
    p = fma(p, r, q.c[0]);
    p = fma(p, r, 1.0);
#if defined(__HIP_DEVICE_COMPILE__)
    const int k = (int)kd;               // the conversion instruction gives 0 for a NaN
#else
    const int k = kd == kd ? (int)kd : 0;
#endif
    const double s = u2d((uint64_t)(1023 + k) << 52);          // 2^k, 0 <= k <= 58
    const double em1 = fma(s, r * p, s - 1.0);
    const float t = (float)(em1 / (em1 + 2.0));                // NaN for a NaN argument
    return copysignf(t, x);
}
ZM_HD float tanhf_ulp2(float x) { return tanhf_ulp2(x, TanhUlp2Coef()); }

// the f32 restatements above with their tables at hand
ZM_HD float expf_glibc(float x) { return expf_glibc(x, exp2f_table()); }
ZM_HD float logf_glibc(float x) { return logf_glibc(x, logf_table()); }
ZM_HD float powf_glibc(float x, float y) { return powf_glibc(x, y, exp2f_table(), powf_log2_table()); }
// sinhf for 64-wide execution, in the manner of tanhf_simd_core: expm1(|x|) with one path through
// the argument reduction and the rational core, the tails k = 0, k = 1 (both of its forms) and
// 2 <= k <= 22 side by side, one quotient for both of sinh's ranges; |x| >= 15.5 (k could reach 23),
// infinities and NaN go to sinhf_fdlibm.  Same results as sinhf_fdlibm on every f32 bit pattern.
ZM_RARE float sinhf_rare(float x, const uint64_t *etab) { return sinhf_fdlibm(x, etab); }
ZM_RARE float coshf_rare(float x, const uint64_t *etab) { return coshf_fdlibm(x, etab); }

ZM_HD float sinhf_simd(float x, const uint64_t *etab, const TanhRegs &rg = TanhRegs())
{
    const float one = 1.0f;
    const float ln2_hi = u2f(0x3f317180u), ln2_lo = u2f(0x3717f7d1u), invln2 = u2f(0x3fb8aa3bu);
    const float Q1 = u2f(0xbd088889u), Q2 = u2f(0x3ad00d01u), Q3 = u2f(0xb8a670cdu), Q5 = u2f(0xb457edbbu);
    const float a = u2f(f2u(x) & 0x7fffffffu);
    if (__builtin_expect(!(a < 15.5f), 0)) return sinhf_rare(x, etab);

    // k = trunc(a/ln2 + 0.5) in one fused step (ties go up, as in fdlibm; rounding a/ln2 to the
    // nearest even integer instead changes one result)
    const float tk = __builtin_floorf(__builtin_fmaf(invln2, a, 0.5f));
    const uint32_t kb = (uint32_t)(int32_t)tk;   // 0 <= k <= 22
#if defined(__HIP_DEVICE_COMPILE__)
    const float hi = __builtin_fmaf(-tk, ln2_hi, a);
#else
    const float hi = a - tk * ln2_hi;        // the product is exact: same value
#endif
    const float lo = tk * ln2_lo;
    const float xr = hi - lo;
    const float c = (hi - xr) - lo;
    const float hfx = 0.5f * xr;
    const float hxs = xr * hfx;
    float sp = __builtin_fmaf(hxs, Q5, rg.q4);
    sp = __builtin_fmaf(hxs, sp, Q3);
    sp = __builtin_fmaf(hxs, sp, Q2);
    sp = __builtin_fmaf(hxs, sp, Q1);
    const float r1 = one + hxs * sp;
    const float t = 3.0f - r1 * hfx;
    const float e = hxs * div_tanh(r1 - t, 6.0f - xr * t);
    float e1 = xr * (e - c) - c;
    e1 -= hxs;
    const float d = e1 - xr;
    // k == 1: 1 + 2 (xr - e1), or -2 (e1 - (xr + 0.5)) when xr < -0.25; the doublings are exact
#if defined(__HIP_DEVICE_COMPILE__)
    const float k1b = __builtin_fmaf(-2.0f, d, one);
#else
    const float k1b = one + 2.0f * (xr - e1);
#endif
    const float k1a = -2.0f * (e1 - (xr + 0.5f));
    const float k1 = (xr < -0.25f) ? k1a : k1b;
    const float tt = u2f(0x3f800000u - (0x1000000u >> (kb & 31)));
    const float y = tt - d;
    float em1 = u2f(f2u(y) + (kb << 23));
    em1 = (kb == 1u) ? k1 : em1;
    em1 = (kb == 0u) ? -d : em1;                        // k == 0 (c is 0: xr - (xr e - hxs) = -d)

    // |x| < 1: h (2t - t t/(t+1));  else h (t + t/(t+1)), h = +-0.5
    const bool small = a < one;
    const float q = div_tanh(small ? em1 * em1 : em1, em1 + one);
#if defined(__HIP_DEVICE_COMPILE__)
    const float r = small ? __builtin_fmaf(2.0f, em1, -q) : em1 + q;
#else
    const float r = small ? 2.0f * em1 - q : em1 + q;
#endif
    return u2f(f2u(0.5f * r) | (f2u(x) & 0x80000000u));
}

// coshf with the same means: below 0.5 ln2 expm1's k = 0 path (no argument reduction), from there to
// 22 expf; the quotients are div_tanh's.  |x| >= 22, infinities and NaN go to coshf_fdlibm.
ZM_HD float coshf_simd(float x, const uint64_t *etab, const TanhRegs &rg = TanhRegs(), const ExpfCoef &ek = ExpfCoef())
{
    const float one = 1.0f, half = 0.5f;
    const float a = u2f(f2u(x) & 0x7fffffffu);
    if (__builtin_expect(!(a < 22.0f), 0)) return coshf_rare(x, etab);
    if (a < u2f(0x3eb17218u)) {
        const float Q1 = u2f(0xbd088889u), Q2 = u2f(0x3ad00d01u), Q3 = u2f(0xb8a670cdu), Q5 = u2f(0xb457edbbu);
        const float hfx = half * a;
        const float hxs = a * hfx;
        float sp = __builtin_fmaf(hxs, Q5, rg.q4);
        sp = __builtin_fmaf(hxs, sp, Q3);
        sp = __builtin_fmaf(hxs, sp, Q2);
        sp = __builtin_fmaf(hxs, sp, Q1);
        const float r1 = one + hxs * sp;
        const float t3 = 3.0f - r1 * hfx;
        const float e = hxs * div_tanh(r1 - t3, 6.0f - a * t3);
        const float t = a - (a * e - hxs);
        const float w = one + t;
        return one + div_tanh(t * t, w + w);
    }
    // 0.34 <= a < 22: expf's main path without its range checks, its f64 constants from the caller
    // (a kernel holds them in scalar registers; as literals each costs two scalar moves per use)
    const float t = expf_glibc_core(a, etab, ek);
    return half * t + div_tanh(half, t);
}

ZM_HD float sinhf_fdlibm(float x) { return sinhf_fdlibm(x, exp2f_table()); }
ZM_HD float coshf_fdlibm(float x) { return coshf_fdlibm(x, exp2f_table()); }

// ---- double precision log: the table-driven routine glibc ships since 2.28 (from ARM's optimized routines) ----
// x = 2^k z, z in [0.6875, 1.375) in 128 subintervals (80 of 1/256 below 1, 48 of 1/128 above); with c near the
// centre of z's subinterval, log(x) = k ln2 + log(c) + log1p(z/c - 1): r = z invc - 1 by one fused multiply-add,
// k ln2_hi + logc exact (logc and ln2_hi are multiples of 2^-43), a degree-5 polynomial in r.  Arguments in
// [1 - 2^-4, 1 + 0x1.09p-4) take a degree-11 polynomial in x - 1 instead, with r - r^2/2 carried in two parts.
// The table {invc, logc} is not defined by a formula: its authors tried the 2^30 doubles around 1 / centre as
// invc and kept one whose log(c), c = 1 / invc, lies within 2^-66 of a multiple of 2^-43 (and which meets
// further conditions of the build without fused multiply-add).  It is rebuilt here along that construction
// (tablegen/log64_table.cpp): every invc of that range whose log(c) is that close to the grid -- about 420
// per subinterval -- is a candidate, and the candidate that gives the host libm's bits on 10^5 random
// arguments of its subinterval is the entry; for every subinterval exactly one does.  The polynomial
// coefficients and the split of ln2 are the sources' constants.  Fused multiply-adds as in the x86-64
// build that CPUs with FMA select (every a + b c, including y = r^3 p + lo in the branch near 1).
// Equal to the host libm's log on 8e8 sampled arguments (uniform bit patterns, [0.5, 1.5), [0, 100), and
// log-uniform over +-700), zero, negative, infinite and subnormal arguments included.
#define ZM_LOG64_TAB                                                                                        \
    {                                                                                                       \
      0x3ff734f0c3e0de9full, 0xbfd7cc7f79e69000ull, 0x3ff713786a2ce91full, 0xbfd76feec20d0000ull,           \
      0x3ff6f26008fab5a0ull, 0xbfd713e31351e000ull, 0x3ff6d1a61f138c7dull, 0xbfd6b85b38287800ull,           \
      0x3ff6b1490bc5b4d1ull, 0xbfd65d5590807800ull, 0x3ff69147332f0cbaull, 0xbfd602d076180000ull,           \
      0x3ff6719f18224223ull, 0xbfd5a8ca86909000ull, 0x3ff6524f99a51ed9ull, 0xbfd54f4356035000ull,           \
      0x3ff63356aa8f24c4ull, 0xbfd4f637c36b4000ull, 0x3ff614b36b9ddc14ull, 0xbfd49da7fda85000ull,           \
      0x3ff5f66452c65c4cull, 0xbfd445923989a800ull, 0x3ff5d867b5912c4full, 0xbfd3edf439b0b800ull,           \
      0x3ff5babccb5b90deull, 0xbfd396ce448f7000ull, 0x3ff59d61f2d91a78ull, 0xbfd3401e17bda000ull,           \
      0x3ff5805612465687ull, 0xbfd2e9e2ef468000ull, 0x3ff56397cee76bd3ull, 0xbfd2941b3830e000ull,           \
      0x3ff54725e2a77f93ull, 0xbfd23ec58cda8800ull, 0x3ff52aff42064583ull, 0xbfd1e9e129279000ull,           \
      0x3ff50f22dbb2bddfull, 0xbfd1956d2b48f800ull, 0x3ff4f38f4734ded7ull, 0xbfd141679ab9f800ull,           \
      0x3ff4d843cfde2840ull, 0xbfd0edd094ef9800ull, 0x3ff4bd3ec078a3c8ull, 0xbfd09aa518db1000ull,           \
      0x3ff4a27fc3e0258aull, 0xbfd047e65263b800ull, 0x3ff4880524d48434ull, 0xbfcfeb224586f000ull,           \
      0x3ff46dce1b192d0bull, 0xbfcf474a7517b000ull, 0x3ff453d9d3391854ull, 0xbfcea4443d103000ull,           \
      0x3ff43a2744b4845aull, 0xbfce020d44e9b000ull, 0x3ff420b54115f8fbull, 0xbfcd60a22977f000ull,           \
      0x3ff40782da3ef4b1ull, 0xbfccc00104959000ull, 0x3ff3ee8f5d57fe8full, 0xbfcc202956891000ull,           \
      0x3ff3d5d9a00b4ce9ull, 0xbfcb81178d811000ull, 0x3ff3bd60c010c12bull, 0xbfcae2c9ccd3d000ull,           \
      0x3ff3a5242b75dab8ull, 0xbfca45402e129000ull, 0x3ff38d22cd9fd002ull, 0xbfc9a877681df000ull,           \
      0x3ff3755bc5847a1cull, 0xbfc90c6d69483000ull, 0x3ff35dce49ad36e2ull, 0xbfc87120a645c000ull,           \
      0x3ff34679984dd440ull, 0xbfc7d68fb4143000ull, 0x3ff32f5cceffcb24ull, 0xbfc73cb83c627000ull,           \
      0x3ff3187775a10d49ull, 0xbfc6a39a9b376000ull, 0x3ff301c8373e3990ull, 0xbfc60b3154b7a000ull,           \
      0x3ff2eb4ebb95f841ull, 0xbfc5737d76243000ull, 0x3ff2d50a0219a9d1ull, 0xbfc4dc7b8fc23000ull,           \
      0x3ff2bef9a8b7fd2aull, 0xbfc4462c51d20000ull, 0x3ff2a91c7a0c1babull, 0xbfc3b08abc830000ull,           \
      0x3ff293726014b530ull, 0xbfc31b996b490000ull, 0x3ff27dfa5757a1f5ull, 0xbfc2875490a44000ull,           \
      0x3ff268b39b1d3bbfull, 0xbfc1f3b9f879a000ull, 0x3ff2539d838ff5bdull, 0xbfc160c8252ca000ull,           \
      0x3ff23eb7aac9083bull, 0xbfc0ce7f57f72000ull, 0x3ff22a012ba940b6ull, 0xbfc03cdc49fea000ull,           \
      0x3ff2157996cc4132ull, 0xbfbf57bdbc4b8000ull, 0x3ff201201dd2fc9bull, 0xbfbe370896404000ull,           \
      0x3ff1ecf4494d480bull, 0xbfbd17983ef94000ull, 0x3ff1d8f5528f6569ull, 0xbfbbf9674ed8a000ull,           \
      0x3ff1c52311577e7cull, 0xbfbadc79202f6000ull, 0x3ff1b17c74cb26e9ull, 0xbfb9c0c3e7288000ull,           \
      0x3ff19e010c2c1ab6ull, 0xbfb8a646b372c000ull, 0x3ff18ab07bb670bdull, 0xbfb78d01b3ac0000ull,           \
      0x3ff1778a25efbcb6ull, 0xbfb674f145380000ull, 0x3ff1648d354c31daull, 0xbfb55e0e6d878000ull,           \
      0x3ff151b990275fddull, 0xbfb4485cdea1e000ull, 0x3ff13f0ea432d24cull, 0xbfb333d94d6aa000ull,           \
      0x3ff12c8b7210f9daull, 0xbfb22079f8c56000ull, 0x3ff11a3028ecb531ull, 0xbfb10e4698622000ull,           \
      0x3ff107fbda8434afull, 0xbfaffa6c6ad20000ull, 0x3ff0f5ee0f4e6bb3ull, 0xbfadda8d4a774000ull,           \
      0x3ff0e4065d2a9fceull, 0xbfabbcece4850000ull, 0x3ff0d244632ca521ull, 0xbfa9a1894012c000ull,           \
      0x3ff0c0a77ce2981aull, 0xbfa788583302c000ull, 0x3ff0af2f83c636d1ull, 0xbfa5715e67d68000ull,           \
      0x3ff09ddb98a01339ull, 0xbfa35c8a49658000ull, 0x3ff08cabaf52e7dfull, 0xbfa149e364154000ull,           \
      0x3ff07b9f2f4e28fbull, 0xbf9e72c082eb8000ull, 0x3ff06ab58c358f19ull, 0xbf9a55f152528000ull,           \
      0x3ff059eea5ecf92cull, 0xbf963d62cf818000ull, 0x3ff04949cdd12c90ull, 0xbf9228fb8caa0000ull,           \
      0x3ff038c6c6f0ada9ull, 0xbf8c317b20f90000ull, 0x3ff02865137932a9ull, 0xbf8419355daa0000ull,           \
      0x3ff0182427ea7348ull, 0xbf781203c2ec0000ull, 0x3ff008040614b195ull, 0xbf60040979240000ull,           \
      0x3fefe01ff726fa1aull, 0x3f6feff384900000ull, 0x3fefa11cc261ea74ull, 0x3f87dc41353d0000ull,           \
      0x3fef6310b081992eull, 0x3f93cea3c4c28000ull, 0x3fef25f63ceeadcdull, 0x3f9b9fc114890000ull,           \
      0x3feee9c8039113e7ull, 0x3fa1b0d8ce110000ull, 0x3feeae8078cbb1abull, 0x3fa58a5bd001c000ull,           \
      0x3fee741aa29d0c9bull, 0x3fa95c8340d88000ull, 0x3fee3a91830a99b5ull, 0x3fad276aef578000ull,           \
      0x3fee01e009609a56ull, 0x3fb07598e598c000ull, 0x3fedca01e577bb98ull, 0x3fb253f5e30d2000ull,           \
      0x3fed92f20b7c9103ull, 0x3fb42edd8b380000ull, 0x3fed5cac66fb5cceull, 0x3fb606598757c000ull,           \
      0x3fed272caa5ede9dull, 0x3fb7da76356a0000ull, 0x3fecf26e3e6b2ccdull, 0x3fb9ab434e1c6000ull,           \
      0x3fecbe6da2a77902ull, 0x3fbb78c7bb0d6000ull, 0x3fec8b266d37086dull, 0x3fbd431332e72000ull,           \
      0x3fec5894bd5d5804ull, 0x3fbf0a3171de6000ull, 0x3fec26b533bb9f8cull, 0x3fc067152b914000ull,           \
      0x3febf583eeece73full, 0x3fc147858292b000ull, 0x3febc4fd75db96c1ull, 0x3fc2266ecdca3000ull,           \
      0x3feb951e0c864a28ull, 0x3fc303d7a6c55000ull, 0x3feb65e2c5ef3e2cull, 0x3fc3dfc33c331000ull,           \
      0x3feb374867c9888bull, 0x3fc4ba366b7a8000ull, 0x3feb094b211d304aull, 0x3fc5933928d1f000ull,           \
      0x3feadbe885f2ef7eull, 0x3fc66acd2418f000ull, 0x3feaaf1d31603da2ull, 0x3fc740f8ec669000ull,           \
      0x3fea82e63fd358a7ull, 0x3fc815c0f51af000ull, 0x3fea5740ef09738bull, 0x3fc8e92954f68000ull,           \
      0x3fea2c2a90ab4b27ull, 0x3fc9bb3602f84000ull, 0x3fea01a01393f2d1ull, 0x3fca8bed1c2c0000ull,           \
      0x3fe9d79f24db3c1bull, 0x3fcb5b515c01d000ull, 0x3fe9ae2505c7b190ull, 0x3fcc2967ccbcc000ull,           \
      0x3fe9852ef297ce2full, 0x3fccf635d5486000ull, 0x3fe95cbaeea44b75ull, 0x3fcdc1bd3446c000ull,           \
      0x3fe934c69de74838ull, 0x3fce8c01b8cfe000ull, 0x3fe90d4f2f6752e6ull, 0x3fcf5509c0179000ull,           \
      0x3fe8e6528effd79dull, 0x3fd00e6c121fb800ull, 0x3fe8bfce9fcc007cull, 0x3fd071b80e93d000ull,           \
      0x3fe899c0dabec30eull, 0x3fd0d46b9e867000ull, 0x3fe87427aa2317fbull, 0x3fd13687334bd000ull,           \
      0x3fe84f00acb39a08ull, 0x3fd1980d67234800ull, 0x3fe82a49e8653e55ull, 0x3fd1f8ffe0cc8000ull,           \
      0x3fe8060195f40260ull, 0x3fd2595fd7636800ull, 0x3fe7e22563e0a329ull, 0x3fd2b9300914a800ull,           \
      0x3fe7beb377dcb5adull, 0x3fd3187210436000ull, 0x3fe79baa679725c2ull, 0x3fd377266dec1800ull,           \
      0x3fe77907f2170657ull, 0x3fd3d54ffbaf3000ull, 0x3fe756cadbd6130cull, 0x3fd432eee32fe000ull            \
    }
static const uint64_t kLog64TabHost[256] = ZM_LOG64_TAB;
#if defined(__HIPCC__)
static __device__ const uint64_t kLog64TabDev[256] = ZM_LOG64_TAB;
#endif
ZM_HD const double *log64_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return reinterpret_cast<const double *>(kLog64TabDev);
#else
    return reinterpret_cast<const double *>(kLog64TabHost);
#endif
}

// the constants as data (a kernel argument: scalar registers feed the f64 operations directly)
struct LogCoef64 {
    double a0 = -0x1.0000000000001p-1, a1 = 0x1.555555551305bp-2, a2 = -0x1.fffffffeb459p-3, a3 = 0x1.999b324f10111p-3,
           a4 = -0x1.55575e506c89fp-3;
    double b1 = 0x1.5555555555577p-2, b2 = -0x1.ffffffffffdcbp-3, b3 = 0x1.999999995dd0cp-3, b4 = -0x1.55555556745a7p-3,
           b5 = 0x1.24924a344de3p-3, b6 = -0x1.fffffa4423d65p-4, b7 = 0x1.c7184282ad6cap-4, b8 = -0x1.999eb43b068ffp-4,
           b9 = 0x1.78182f7afd085p-4, b10 = -0x1.5521375d145cdp-4;
    double ln2hi = 0x1.62e42fefa3800p-1, ln2lo = 0x1.ef35793c76730p-45;
};

ZM_HD double log_glibc(double x, const double *tab, const LogCoef64 &k = LogCoef64())
{
    uint64_t ix = d2u(x);
    const uint64_t lo1 = 0x3fee000000000000ull, hi1 = 0x3ff1090000000000ull;   // 1 - 2^-4, 1 + 0x1.09p-4
    if (ix - lo1 < hi1 - lo1) {
        if (ix == 0x3ff0000000000000ull) return 0.0;
        const double r = x - 1.0, r2 = r * r, r3 = r * r2;
        const double p3 = __builtin_fma(r3, k.b10, __builtin_fma(r2, k.b9, __builtin_fma(r, k.b8, k.b7)));
        const double p2 = __builtin_fma(r3, p3, __builtin_fma(r2, k.b6, __builtin_fma(r, k.b5, k.b4)));
        const double p1 = __builtin_fma(r3, p2, __builtin_fma(r2, k.b3, __builtin_fma(r, k.b2, k.b1)));
        // r - r^2 / 2 as hi + lo: r split at 2^-27 relative, so that the square of the high part is exact
        double w = r * 0x1p27;
        const double rhi = r + w - w, rlo = r - rhi;
        w = rhi * rhi * -0.5;
        const double hi = r + w;
        double lo = r - hi + w;
        lo = __builtin_fma(-0.5 * rlo, rhi + r, lo);
        return __builtin_fma(r3, p1, lo) + hi;
    }
    const uint32_t top = (uint32_t)(ix >> 48);
    if (__builtin_expect(top - 0x0010u >= 0x7ff0u - 0x0010u, 0)) {
        if (ix * 2 == 0) return -u2d(0x7ff0000000000000ull);                  // log(+-0) = -inf
        if (ix == 0x7ff0000000000000ull) return x;                             // log(inf) = inf
        if ((top & 0x8000u) || (top & 0x7ff0u) == 0x7ff0u) return (x - x) * u2d(0x7ff0000000000000ull);   // negative, NaN
        ix = d2u(x * 0x1p52);                                                  // subnormal: normalise
        ix -= 52ull << 52;
    }
    const uint64_t tmp = ix - 0x3fe6000000000000ull;
    const int i = (int)((tmp >> 45) & 127u);
    const int64_t ke = (int64_t)tmp >> 52;
    const double z = u2d(ix - (tmp & (0xfffull << 52)));
    const double invc = tab[2 * i], logc = tab[2 * i + 1];
    const double r = __builtin_fma(z, invc, -1.0);
    const double kd = (double)ke;
    const double w = __builtin_fma(kd, k.ln2hi, logc);
    const double hi = w + r;
    const double lo = __builtin_fma(kd, k.ln2lo, (w - hi) + r);
    const double r2 = r * r;
    const double p = __builtin_fma(r2, __builtin_fma(r, k.a4, k.a3), __builtin_fma(r, k.a2, k.a1));
    double y = __builtin_fma(r2, k.a0, lo);
    y = __builtin_fma(r * r2, p, y);
    return y + hi;
}
ZM_HD double log_glibc(double x) { return log_glibc(x, log64_table()); }

// ---- double precision pow: the routine glibc ships since 2.28 (from ARM's optimized routines) -----------
// log(x) as hi + lo to about 68 bits -- x = 2^k z, z in [0x1.69555p-1, 0x1.69555p0) in 128 subintervals, 1 / c a
// multiple of 1/128 resp. 1/256 so that r = z / c - 1 is exact, k ln2 + log(c) + r - r^2 / 2 carried in two
// doubles, a degree-7 polynomial for the rest -- then y log(x) as ehi + elo and exp of that through exp's
// table with the tail added to the reduced argument and the sign of a negative base (odd integer y) carried
// in the scale.  The log table IS defined by a formula (tablegen/pow64_table.py rebuilds it with exact
// rational arithmetic: invc = the nearest multiple, logc = log(c) rounded to a multiple of 2^-43, logctail =
// the nearest double of the rest); the polynomial and the split of ln2 are the sources' constants.  Fused
// multiply-adds as in the x86-64 build that CPUs with FMA select: every a + b c, including the polynomial's
// last product into the sum of the low parts.  Equal to the host libm's pow on 1.6e8 sampled pairs: uniform bit
// patterns for both arguments, bases in [0, 4) with exponents in +-40, bases in [0.5, 1.5) with exponents in
// +-1000, log-uniform and negative bases under sixteen fixed exponents.
#define ZM_POW64_LOG_TAB                                                                                    \
    {                                                                                                       \
      0x3ff6a00000000000ull, 0xbfd62c82f2b9c800ull, 0x3cfab42428375680ull,                                  \
      0x3ff6800000000000ull, 0xbfd5d1bdbf580800ull, 0xbd1ca508d8e0f720ull,                                  \
      0x3ff6600000000000ull, 0xbfd5767717455800ull, 0xbd2362a4d5b6506dull,                                  \
      0x3ff6400000000000ull, 0xbfd51aad872df800ull, 0xbce684e49eb067d5ull,                                  \
      0x3ff6200000000000ull, 0xbfd4be5f95777800ull, 0xbd041b6993293ee0ull,                                  \
      0x3ff6000000000000ull, 0xbfd4618bc21c6000ull, 0x3d13d82f484c84ccull,                                  \
      0x3ff5e00000000000ull, 0xbfd404308686a800ull, 0x3cdc42f3ed820b3aull,                                  \
      0x3ff5c00000000000ull, 0xbfd3a64c55694800ull, 0x3d20b1c686519460ull,                                  \
      0x3ff5a00000000000ull, 0xbfd347dd9a988000ull, 0x3d25594dd4c58092ull,                                  \
      0x3ff5800000000000ull, 0xbfd2e8e2bae12000ull, 0x3d267b1e99b72bd8ull,                                  \
      0x3ff5600000000000ull, 0xbfd2895a13de8800ull, 0x3d15ca14b6cfb03full,                                  \
      0x3ff5600000000000ull, 0xbfd2895a13de8800ull, 0x3d15ca14b6cfb03full,                                  \
      0x3ff5400000000000ull, 0xbfd22941fbcf7800ull, 0xbd165a242853da76ull,                                  \
      0x3ff5200000000000ull, 0xbfd1c898c1699800ull, 0xbd1fafbc68e75404ull,                                  \
      0x3ff5000000000000ull, 0xbfd1675cababa800ull, 0x3d1f1fc63382a8f0ull,                                  \
      0x3ff4e00000000000ull, 0xbfd1058bf9ae4800ull, 0xbd26a8c4fd055a66ull,                                  \
      0x3ff4c00000000000ull, 0xbfd0a324e2739000ull, 0xbd0c6bee7ef4030eull,                                  \
      0x3ff4a00000000000ull, 0xbfd0402594b4d000ull, 0xbcf036b89ef42d7full,                                  \
      0x3ff4a00000000000ull, 0xbfd0402594b4d000ull, 0xbcf036b89ef42d7full,                                  \
      0x3ff4800000000000ull, 0xbfcfb9186d5e4000ull, 0x3d0d572aab993c87ull,                                  \
      0x3ff4600000000000ull, 0xbfcef0adcbdc6000ull, 0x3d2b26b79c86af24ull,                                  \
      0x3ff4400000000000ull, 0xbfce27076e2af000ull, 0xbd172f4f543fff10ull,                                  \
      0x3ff4200000000000ull, 0xbfcd5c216b4fc000ull, 0x3d21ba91bbca681bull,                                  \
      0x3ff4000000000000ull, 0xbfcc8ff7c79aa000ull, 0x3d27794f689f8434ull,                                  \
      0x3ff4000000000000ull, 0xbfcc8ff7c79aa000ull, 0x3d27794f689f8434ull,                                  \
      0x3ff3e00000000000ull, 0xbfcbc286742d9000ull, 0x3d194eb0318bb78full,                                  \
      0x3ff3c00000000000ull, 0xbfcaf3c94e80c000ull, 0x3cba4e633fcd9066ull,                                  \
      0x3ff3a00000000000ull, 0xbfca23bc1fe2b000ull, 0xbd258c64dc46c1eaull,                                  \
      0x3ff3a00000000000ull, 0xbfca23bc1fe2b000ull, 0xbd258c64dc46c1eaull,                                  \
      0x3ff3800000000000ull, 0xbfc9525a9cf45000ull, 0xbd2ad1d904c1d4e3ull,                                  \
      0x3ff3600000000000ull, 0xbfc87fa06520d000ull, 0x3d2bbdbf7fdbfa09ull,                                  \
      0x3ff3400000000000ull, 0xbfc7ab890210e000ull, 0x3d2bdb9072534a58ull,                                  \
      0x3ff3400000000000ull, 0xbfc7ab890210e000ull, 0x3d2bdb9072534a58ull,                                  \
      0x3ff3200000000000ull, 0xbfc6d60fe719d000ull, 0xbd10e46aa3b2e266ull,                                  \
      0x3ff3000000000000ull, 0xbfc5ff3070a79000ull, 0xbd1e9e439f105039ull,                                  \
      0x3ff3000000000000ull, 0xbfc5ff3070a79000ull, 0xbd1e9e439f105039ull,                                  \
      0x3ff2e00000000000ull, 0xbfc526e5e3a1b000ull, 0xbd20de8b90075b8full,                                  \
      0x3ff2c00000000000ull, 0xbfc44d2b6ccb8000ull, 0x3d170cc16135783cull,                                  \
      0x3ff2c00000000000ull, 0xbfc44d2b6ccb8000ull, 0x3d170cc16135783cull,                                  \
      0x3ff2a00000000000ull, 0xbfc371fc201e9000ull, 0x3cf178864d27543aull,                                  \
      0x3ff2800000000000ull, 0xbfc29552f81ff000ull, 0xbd248d301771c408ull,                                  \
      0x3ff2600000000000ull, 0xbfc1b72ad52f6000ull, 0xbd2e80a41811a396ull,                                  \
      0x3ff2600000000000ull, 0xbfc1b72ad52f6000ull, 0xbd2e80a41811a396ull,                                  \
      0x3ff2400000000000ull, 0xbfc0d77e7cd09000ull, 0x3d0a699688e85bf4ull,                                  \
      0x3ff2400000000000ull, 0xbfc0d77e7cd09000ull, 0x3d0a699688e85bf4ull,                                  \
      0x3ff2200000000000ull, 0xbfbfec9131dbe000ull, 0xbd2575545ca333f2ull,                                  \
      0x3ff2000000000000ull, 0xbfbe27076e2b0000ull, 0x3d2a342c2af0003cull,                                  \
      0x3ff2000000000000ull, 0xbfbe27076e2b0000ull, 0x3d2a342c2af0003cull,                                  \
      0x3ff1e00000000000ull, 0xbfbc5e548f5bc000ull, 0xbd1d0c57585fbe06ull,                                  \
      0x3ff1c00000000000ull, 0xbfba926d3a4ae000ull, 0x3d253935e85baac8ull,                                  \
      0x3ff1c00000000000ull, 0xbfba926d3a4ae000ull, 0x3d253935e85baac8ull,                                  \
      0x3ff1a00000000000ull, 0xbfb8c345d631a000ull, 0x3d137c294d2f5668ull,                                  \
      0x3ff1a00000000000ull, 0xbfb8c345d631a000ull, 0x3d137c294d2f5668ull,                                  \
      0x3ff1800000000000ull, 0xbfb6f0d28ae56000ull, 0xbd269737c93373daull,                                  \
      0x3ff1600000000000ull, 0xbfb51b073f062000ull, 0x3d1f025b61c65e57ull,                                  \
      0x3ff1600000000000ull, 0xbfb51b073f062000ull, 0x3d1f025b61c65e57ull,                                  \
      0x3ff1400000000000ull, 0xbfb341d7961be000ull, 0x3d2c5edaccf913dfull,                                  \
      0x3ff1400000000000ull, 0xbfb341d7961be000ull, 0x3d2c5edaccf913dfull,                                  \
      0x3ff1200000000000ull, 0xbfb16536eea38000ull, 0x3d147c5e768fa309ull,                                  \
      0x3ff1000000000000ull, 0xbfaf0a30c0118000ull, 0x3d2d599e83368e91ull,                                  \
      0x3ff1000000000000ull, 0xbfaf0a30c0118000ull, 0x3d2d599e83368e91ull,                                  \
      0x3ff0e00000000000ull, 0xbfab42dd71198000ull, 0x3d1c827ae5d6704cull,                                  \
      0x3ff0e00000000000ull, 0xbfab42dd71198000ull, 0x3d1c827ae5d6704cull,                                  \
      0x3ff0c00000000000ull, 0xbfa77458f632c000ull, 0xbd2cfc4634f2a1eeull,                                  \
      0x3ff0c00000000000ull, 0xbfa77458f632c000ull, 0xbd2cfc4634f2a1eeull,                                  \
      0x3ff0a00000000000ull, 0xbfa39e87b9fec000ull, 0x3cf502b7f526feaaull,                                  \
      0x3ff0a00000000000ull, 0xbfa39e87b9fec000ull, 0x3cf502b7f526feaaull,                                  \
      0x3ff0800000000000ull, 0xbf9f829b0e780000ull, 0xbd2980267c7e09e4ull,                                  \
      0x3ff0800000000000ull, 0xbf9f829b0e780000ull, 0xbd2980267c7e09e4ull,                                  \
      0x3ff0600000000000ull, 0xbf97b91b07d58000ull, 0xbd288d5493faa639ull,                                  \
      0x3ff0400000000000ull, 0xbf8fc0a8b0fc0000ull, 0xbcdf1e7cf6d3a69cull,                                  \
      0x3ff0400000000000ull, 0xbf8fc0a8b0fc0000ull, 0xbcdf1e7cf6d3a69cull,                                  \
      0x3ff0200000000000ull, 0xbf7fe02a6b100000ull, 0xbd19e23f0dda40e4ull,                                  \
      0x3ff0200000000000ull, 0xbf7fe02a6b100000ull, 0xbd19e23f0dda40e4ull,                                  \
      0x3ff0000000000000ull, 0x0000000000000000ull, 0x0000000000000000ull,                                  \
      0x3ff0000000000000ull, 0x0000000000000000ull, 0x0000000000000000ull,                                  \
      0x3fefc00000000000ull, 0x3f80101575890000ull, 0xbd10c76b999d2be8ull,                                  \
      0x3fef800000000000ull, 0x3f90205658938000ull, 0xbd23dc5b06e2f7d2ull,                                  \
      0x3fef400000000000ull, 0x3f98492528c90000ull, 0xbd2aa0ba325a0c34ull,                                  \
      0x3fef000000000000ull, 0x3fa0415d89e74000ull, 0x3d0111c05cf1d753ull,                                  \
      0x3feec00000000000ull, 0x3fa466aed42e0000ull, 0xbd2c167375bdfd28ull,                                  \
      0x3fee800000000000ull, 0x3fa894aa149fc000ull, 0xbd197995d05a267dull,                                  \
      0x3fee400000000000ull, 0x3faccb73cdddc000ull, 0xbd1a68f247d82807ull,                                  \
      0x3fee200000000000ull, 0x3faeea31c006c000ull, 0xbd0e113e4fc93b7bull,                                  \
      0x3fede00000000000ull, 0x3fb1973bd1466000ull, 0xbd25325d560d9e9bull,                                  \
      0x3feda00000000000ull, 0x3fb3bdf5a7d1e000ull, 0x3d2cc85ea5db4ed7ull,                                  \
      0x3fed600000000000ull, 0x3fb5e95a4d97a000ull, 0xbd2c69063c5d1d1eull,                                  \
      0x3fed400000000000ull, 0x3fb700d30aeac000ull, 0x3cec1e8da99ded32ull,                                  \
      0x3fed000000000000ull, 0x3fb9335e5d594000ull, 0x3d23115c3abd47daull,                                  \
      0x3fecc00000000000ull, 0x3fbb6ac88dad6000ull, 0xbd1390802bf768e5ull,                                  \
      0x3feca00000000000ull, 0x3fbc885801bc4000ull, 0x3d2646d1c65aacd3ull,                                  \
      0x3fec600000000000ull, 0x3fbec739830a2000ull, 0xbd2dc068afe645e0ull,                                  \
      0x3fec400000000000ull, 0x3fbfe89139dbe000ull, 0xbd2534d64fa10afdull,                                  \
      0x3fec000000000000ull, 0x3fc1178e8227e000ull, 0x3d21ef78ce2d07f2ull,                                  \
      0x3febe00000000000ull, 0x3fc1aa2b7e23f000ull, 0x3d2ca78e44389934ull,                                  \
      0x3feba00000000000ull, 0x3fc2d1610c868000ull, 0x3d039d6ccb81b4a1ull,                                  \
      0x3feb800000000000ull, 0x3fc365fcb0159000ull, 0x3cc62fa8234b7289ull,                                  \
      0x3feb400000000000ull, 0x3fc4913d8333b000ull, 0x3d25837954fdb678ull,                                  \
      0x3feb200000000000ull, 0x3fc527e5e4a1b000ull, 0x3d2633e8e5697dc7ull,                                  \
      0x3feae00000000000ull, 0x3fc6574ebe8c1000ull, 0x3d19cf8b2c3c2e78ull,                                  \
      0x3feac00000000000ull, 0x3fc6f0128b757000ull, 0xbd25118de59c21e1ull,                                  \
      0x3feaa00000000000ull, 0x3fc7898d85445000ull, 0xbd1c661070914305ull,                                  \
      0x3fea600000000000ull, 0x3fc8beafeb390000ull, 0xbd073d54aae92cd1ull,                                  \
      0x3fea400000000000ull, 0x3fc95a5adcf70000ull, 0x3d07f22858a0ff6full,                                  \
      0x3fea000000000000ull, 0x3fca93ed3c8ae000ull, 0xbd28724350562169ull,                                  \
      0x3fe9e00000000000ull, 0x3fcb31d8575bd000ull, 0xbd0c358d4eace1aaull,                                  \
      0x3fe9c00000000000ull, 0x3fcbd087383be000ull, 0xbd2d4bc4595412b6ull,                                  \
      0x3fe9a00000000000ull, 0x3fcc6ffbc6f01000ull, 0xbcf1ec72c5962bd2ull,                                  \
      0x3fe9600000000000ull, 0x3fcdb13db0d49000ull, 0xbd2aff2af715b035ull,                                  \
      0x3fe9400000000000ull, 0x3fce530effe71000ull, 0x3cc212276041f430ull,                                  \
      0x3fe9200000000000ull, 0x3fcef5ade4dd0000ull, 0xbcca211565bb8e11ull,                                  \
      0x3fe9000000000000ull, 0x3fcf991c6cb3b000ull, 0x3d1bcbecca0cdf30ull,                                  \
      0x3fe8c00000000000ull, 0x3fd07138604d5800ull, 0x3cf89cdb16ed4e91ull,                                  \
      0x3fe8a00000000000ull, 0x3fd0c42d67616000ull, 0x3d27188b163ceae9ull,                                  \
      0x3fe8800000000000ull, 0x3fd1178e8227e800ull, 0xbd2c210e63a5f01cull,                                  \
      0x3fe8600000000000ull, 0x3fd16b5ccbacf800ull, 0x3d2b9acdf7a51681ull,                                  \
      0x3fe8400000000000ull, 0x3fd1bf99635a6800ull, 0x3d2ca6ed5147bdb7ull,                                  \
      0x3fe8200000000000ull, 0x3fd214456d0eb800ull, 0x3d0a87deba46baeaull,                                  \
      0x3fe7e00000000000ull, 0x3fd2bef07cdc9000ull, 0x3d2a9cfa4a5004f4ull,                                  \
      0x3fe7c00000000000ull, 0x3fd314f1e1d36000ull, 0xbd28e27ad3213cb8ull,                                  \
      0x3fe7a00000000000ull, 0x3fd36b6776be1000ull, 0x3d116ecdb0f177c8ull,                                  \
      0x3fe7800000000000ull, 0x3fd3c25277333000ull, 0x3d183b54b606bd5cull,                                  \
      0x3fe7600000000000ull, 0x3fd419b423d5e800ull, 0x3d08e436ec90e09dull,                                  \
      0x3fe7400000000000ull, 0x3fd4718dc271c800ull, 0xbd2f27ce0967d675ull,                                  \
      0x3fe7200000000000ull, 0x3fd4c9e09e173000ull, 0xbd2e20891b0ad8a4ull,                                  \
      0x3fe7000000000000ull, 0x3fd522ae0738a000ull, 0x3d2ebe708164c759ull,                                  \
      0x3fe6e00000000000ull, 0x3fd57bf753c8d000ull, 0x3d1fadedee5d40efull,                                  \
      0x3fe6c00000000000ull, 0x3fd5d5bddf596000ull, 0xbd0a0b2a08a465dcull                                   \
    }
static const uint64_t kPow64LogTabHost[384] = ZM_POW64_LOG_TAB;
#if defined(__HIPCC__)
static __device__ const uint64_t kPow64LogTabDev[384] = ZM_POW64_LOG_TAB;
#endif
ZM_HD const double *pow64_log_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return reinterpret_cast<const double *>(kPow64LogTabDev);
#else
    return reinterpret_cast<const double *>(kPow64LogTabHost);
#endif
}

// the constants as data (a kernel argument: scalar registers feed the f64 operations directly)
struct PowCoef64 {
    double a1 = 0x1.555555555556p-2 * -2, a2 = -0x1.0000000000006p-2 * -2, a3 = 0x1.999999959554ep-3 * 4,
           a4 = -0x1.555555529a47ap-3 * 4, a5 = 0x1.2495b9b4845e9p-3 * -8, a6 = -0x1.0002b8b263fc3p-3 * -8;
    double ln2hi = 0x1.62e42fefa3800p-1, ln2lo = 0x1.ef35793c76730p-45;
    ExpCoef64 e;
};

// log(x) of a positive normal x given by its bits, as the returned high part plus *tail
ZM_HD double pow_log_inline(uint64_t ix, double *tail, const double *ltab, const PowCoef64 &k)
{
    const uint64_t tmp = ix - 0x3fe6955500000000ull;
    const int i = (int)((tmp >> 45) & 127u);
    const int64_t ke = (int64_t)tmp >> 52;
    const double z = u2d(ix - (tmp & (0xfffull << 52)));
    const double kd = (double)ke;
    const double invc = ltab[3 * i], logc = ltab[3 * i + 1], logctail = ltab[3 * i + 2];
    const double r = __builtin_fma(z, invc, -1.0);
    const double t1 = __builtin_fma(kd, k.ln2hi, logc);
    const double t2 = t1 + r;
    const double lo1 = __builtin_fma(kd, k.ln2lo, logctail);
    const double lo2 = t1 - t2 + r;
    const double ar = -0.5 * r, ar2 = r * ar, ar3 = r * ar2;
    const double hi = t2 + ar2;
    const double lo3 = __builtin_fma(ar, r, -ar2);
    const double lo4 = t2 - hi + ar2;
    const double p = __builtin_fma(ar2, __builtin_fma(ar2, __builtin_fma(r, k.a6, k.a5), __builtin_fma(r, k.a4, k.a3)),
                                   __builtin_fma(r, k.a2, k.a1));
    const double lo = __builtin_fma(ar3, p, lo1 + lo2 + lo3 + lo4);
    const double y = hi + lo;
    *tail = hi - y + lo;
    return y;
}

// exp(x + xtail), negated when sign_bias is set (it is added to the scale's exponent field, where it lands on the sign)
ZM_HD double pow_exp_inline(double x, double xtail, uint32_t sign_bias, const uint64_t *etab, const ExpCoef64 &k)
{
    uint32_t abstop = (uint32_t)(d2u(x) >> 52) & 0x7ffu;
    if (abstop - 0x3c9u >= 0x408u - 0x3c9u) {            // |x| < 2^-54 or |x| >= 512
        if (abstop - 0x3c9u >= 0x80000000u) {
            const double one = 1.0 + x;
            return sign_bias ? -one : one;
        }
        if (abstop >= 0x409u) {                          // |x| >= 1024: under- or overflow
            if (d2u(x) >> 63) return sign_bias ? -0.0 : 0.0;
            return u2d(sign_bias ? 0xfff0000000000000ull : 0x7ff0000000000000ull);
        }
        abstop = 0;                                      // large |x|: the special case below
    }
    const double z = k.inv_ln2n * x;
    double kd = z + k.shift;
    const uint64_t ki = d2u(kd);
    kd -= k.shift;
    double r = __builtin_fma(kd, k.neg_ln2lo_n, __builtin_fma(kd, k.neg_ln2hi_n, x));
    r += xtail;
    const uint64_t idx = 2 * (ki % 128);
    const uint64_t top = (ki + sign_bias) << (52 - 7);
    const double tail = u2d(etab[idx]);
    uint64_t sbits = etab[idx + 1] + top;
    const double r2 = r * r;
    const double tmp = __builtin_fma(r2 * r2, __builtin_fma(r, k.c5, k.c4), __builtin_fma(r2, __builtin_fma(r, k.c3, k.c2), tail + r));
    if (abstop == 0) {
        if ((ki & 0x80000000u) == 0) {                   // k > 0: the exponent of scale may have overflowed
            sbits -= 1009ull << 52;
            const double scale = u2d(sbits);
            return 0x1p1009 * __builtin_fma(scale, tmp, scale);
        }
        sbits += 1022ull << 52;                          // k < 0: care in the subnormal range
        const double scale = u2d(sbits);
        double y = scale + scale * tmp;
        if (__builtin_fabs(y) < 1.0) {
            const double one = y < 0.0 ? -1.0 : 1.0;
            double lo = scale - y + scale * tmp;
            const double hi = one + y;
            lo = one - hi + y + lo;
            y = (hi + lo) - one;
            if (y == 0.0) y = u2d(sbits & 0x8000000000000000ull);
        }
        return 0x1p-1022 * y;
    }
    const double scale = u2d(sbits);
    return __builtin_fma(scale, tmp, scale);
}

// 0: y is not an integer, 1: odd, 2: even
ZM_HD int pow_checkint(uint64_t iy)
{
    const int e = (int)(iy >> 52) & 0x7ff;
    if (e < 0x3ff) return 0;
    if (e > 0x3ff + 52) return 2;
    if (iy & ((1ull << (0x3ff + 52 - e)) - 1)) return 0;
    if (iy & (1ull << (0x3ff + 52 - e))) return 1;
    return 2;
}
ZM_HD bool pow_zeroinfnan(uint64_t i) { return 2 * i - 1 >= 2 * 0x7ff0000000000000ull - 1; }
ZM_HD bool pow_issignaling(uint64_t i) { return 2 * (i ^ 0x0008000000000000ull) > 2 * 0x7ff8000000000000ull; }

ZM_HD double pow_glibc_full(double x, double y, const double *ltab, const uint64_t *etab, const PowCoef64 &k = PowCoef64())
{
    const uint64_t one = 0x3ff0000000000000ull, inf = 0x7ff0000000000000ull;
    uint32_t sign_bias = 0;
    uint64_t ix = d2u(x);
    const uint64_t iy = d2u(y);
    uint32_t topx = (uint32_t)(ix >> 52);
    const uint32_t topy = (uint32_t)(iy >> 52);
    if (topx - 0x001u >= 0x7ffu - 0x001u || (topy & 0x7ffu) - 0x3beu >= 0x43eu - 0x3beu) {
        // x subnormal, zero, negative, infinite or NaN; or |y| < 2^-65, |y| >= 2^63 or NaN
        if (pow_zeroinfnan(iy)) {
            if (2 * iy == 0) return pow_issignaling(ix) ? x + y : 1.0;
            if (ix == one) return pow_issignaling(iy) ? x + y : 1.0;
            if (2 * ix > 2 * inf || 2 * iy > 2 * inf) return x + y;
            if (2 * ix == 2 * one) return 1.0;
            if ((2 * ix < 2 * one) == !(iy >> 63)) return 0.0;   // |x| < 1 && y == inf, or |x| > 1 && y == -inf
            return y * y;
        }
        if (pow_zeroinfnan(ix)) {
            double x2 = x * x;
            if ((ix >> 63) && pow_checkint(iy) == 1) x2 = -x2;
            return (iy >> 63) ? 1 / x2 : x2;
        }
        if (ix >> 63) {                                  // finite x < 0
            const int yint = pow_checkint(iy);
            if (yint == 0) return (x - x) * u2d(inf);    // the sources' (x - x) / (x - x): a NaN
            if (yint == 1) sign_bias = 0x800u << 7;
            ix &= 0x7fffffffffffffffull;
            topx &= 0x7ffu;
        }
        if ((topy & 0x7ffu) - 0x3beu >= 0x43eu - 0x3beu) {
            if (ix == one) return 1.0;
            if ((topy & 0x7ffu) < 0x3beu) return ix > one ? 1.0 + y : 1.0 - y;   // |y| < 2^-65
            return (ix > one) == (topy < 0x800u) ? u2d(inf) : 0.0;
        }
        if (topx == 0) {                                 // subnormal x: normalise
            ix = d2u(x * 0x1p52);
            ix &= 0x7fffffffffffffffull;
            ix -= 52ull << 52;
        }
    }
    double lo;
    const double hi = pow_log_inline(ix, &lo, ltab, k);
    const double ehi = y * hi;
    const double elo = __builtin_fma(y, lo, __builtin_fma(y, hi, -ehi));
    return pow_exp_inline(ehi, elo, sign_bias, etab, k.e);
}
ZM_HD double pow_glibc_full(double x, double y) { return pow_glibc_full(x, y, pow64_log_table(), exp_table()); }
// (builds its own constants: a reference to the caller's would force them into memory there)
ZM_RARE double pow_rare(double x, double y, const double *ltab, const uint64_t *etab) { return pow_glibc_full(x, y, ltab, etab); }

// pow as the kernels call it: the main path as straight-line code (positive normal x, 2^-65 <= |y| < 2^63,
// 2^-54 <= |y log x| < 512: no special case applies, no sign to carry), everything else out of line
ZM_HD double pow_glibc(double x, double y, const double *ltab, const uint64_t *etab, const PowCoef64 &k = PowCoef64())
{
    const uint64_t ix = d2u(x), iy = d2u(y);
    const uint32_t topx = (uint32_t)(ix >> 52), topy = (uint32_t)(iy >> 52);
    if (__builtin_expect(topx - 0x001u >= 0x7ffu - 0x001u || (topy & 0x7ffu) - 0x3beu >= 0x43eu - 0x3beu, 0))
        return pow_rare(x, y, ltab, etab);
    double lo;
    const double hi = pow_log_inline(ix, &lo, ltab, k);
    const double ehi = y * hi;
    const double elo = __builtin_fma(y, lo, __builtin_fma(y, hi, -ehi));
    const uint32_t abstop = (uint32_t)(d2u(ehi) >> 52) & 0x7ffu;
    if (__builtin_expect(abstop - 0x3c9u >= 0x408u - 0x3c9u, 0)) return pow_rare(x, y, ltab, etab);
    const ExpCoef64 &e = k.e;
    const double z = e.inv_ln2n * ehi;
    double kd = z + e.shift;
    const uint64_t ki = d2u(kd);
    kd -= e.shift;
    double r = __builtin_fma(kd, e.neg_ln2lo_n, __builtin_fma(kd, e.neg_ln2hi_n, ehi));
    r += elo;
    const uint64_t idx = 2 * (ki % 128);
    const double tail = u2d(etab[idx]);
    const double scale = u2d(etab[idx + 1] + (ki << (52 - 7)));
    const double r2 = r * r;
    const double tmp = __builtin_fma(r2 * r2, __builtin_fma(r, e.c5, e.c4), __builtin_fma(r2, __builtin_fma(r, e.c3, e.c2), tail + r));
    return __builtin_fma(scale, tmp, scale);
}
ZM_HD double pow_glibc(double x, double y) { return pow_glibc(x, y, pow64_log_table(), exp_table()); }

// ---- double precision sin / cos: s_sin.c and branred.c as glibc 2.35 ships them (the IBM Accurate
// Mathematical Library without its multi-precision fall-backs) ------------------------------------------
// |x| < 2^-26: x resp. 1.  The argument is brought to a in [-pi/4, pi/4] plus a small da and a quadrant n:
//   * |x| < 0.855469: a = x;
//   * |x| < 2.426265: a = pi/2 - |x| (sin: da = the low part of pi/2; cos: a and da renormalised);
//   * |x| < 105414350: x - n pi/2 in three pieces of pi/2 (27, 26 and 52 + bits), n from a round-to-integer add;
//   * above: 2/pi in 24-bit pieces times the two 27-bit halves of x, six pieces each from the one that
//     reaches the binary point, the integer parts dropped (branred.c).
// sine (even n) on |a| < 0.126 is a degree-11 Taylor form; otherwise sine and cosine (odd n) come from
// sin(xi), cos(xi) at xi = k/128 (the nearest multiple, read off a + 1.5 2^45), each as a double and the
// double of the remainder, and short polynomials in a - xi, combined by the angle-sum formulas with the
// small terms first.  The table is regenerated here from that definition (exact rational arithmetic:
// tablegen/sincos64_tables.py).
// Fused multiply-adds where the compiler fuses them in the x86-64 build that CPUs with FMA select
// (s_sin.c has one; branred.c has none, and its products are exact anyway).  Equal to the host libm's
// sin and cos on 6.4e8 sampled arguments each: uniform in +-0.855, +-2.43, +-10, +-1000, +-1e6, +-1.05e8,
// +-1e-3, +-1e-9, and random mantissas under every exponent from 2^26 to 2^1023.
// (The library's sincos is another function: it reduces |x| < 2.426265 like the larger arguments and
// differs from sin / cos in the last bit on 1 in 1000 of them.)
#define ZM_SINCOS64_TAB                                                                                     \
    {                                                                                                       \
      0x0000000000000000ull, 0x0000000000000000ull, 0x3ff0000000000000ull, 0x0000000000000000ull,           \
      0x3f7fffeaaaaeeeefull, 0xbc1e45e2ec67b77cull, 0x3fefffc000155552ull, 0x3c8f4a01a0196daeull,           \
      0x3f8fffaaaaeeeed5ull, 0xbc02ab639a9f0776ull, 0x3fefff000155549full, 0x3c828a28a03a5ef3ull,           \
      0x3f97ff7001033255ull, 0x3bfefe2b51527336ull, 0x3feffdc006bff7e6ull, 0x3c8ae6dae86977bdull,           \
      0x3f9ffeaaaeeee86full, 0xbc3cd406fb224ae2ull, 0x3feffc00155527d3ull, 0xbc83b54492d89b5bull,           \
      0x3fa3feb2b12d45d5ull, 0x3c34ec54203d1c11ull, 0x3feff9c03414a7baull, 0x3c6991f4be6c59bfull,           \
      0x3fa7fdc01032fba9ull, 0xbc4599bdf46e997aull, 0x3feff7006bfdf99full, 0xbc78b3b560648d5full,           \
      0x3fabfc6d78586dacull, 0x3c18e4fd03dbf236ull, 0x3feff3c0c8103a31ull, 0x3c74856dbddc0e66ull,           \
      0x3faffaaaeeed4edbull, 0xbc42d16d32684b69ull, 0x3feff0015549f4d3ull, 0x3c8328387b99426full,           \
      0x3fb1fc343d808befull, 0xbc5f3d32e6f3be4full, 0x3fefebc222a8ef9full, 0x3c57934934f54c77ull,           \
      0x3fb3facb12d1755bull, 0xbc5921915299468bull, 0x3fefe7034129ef6full, 0xbc6cbf4337c96f97ull,           \
      0x3fb5f911fd10b737ull, 0xbc50184f02be9102ull, 0x3fefe1c4c3c873ebull, 0xbc35a9c9057c4a02ull,           \
      0x3fb7f701032550e4ull, 0x3c3afc2d1800501aull, 0x3fefdc06bf7e6b9bull, 0x3c831902b535f8dbull,           \
      0x3fb9f4902d55d1f9ull, 0x3c52696d7eac1dc1ull, 0x3fefd5c94b43e000ull, 0xbc62e768cb4f92f9ull,           \
      0x3fbbf1b78568391dull, 0x3c5e91841dea4cc8ull, 0x3fefcf0c800e99b1ull, 0x3c6ea3d786d186acull,           \
      0x3fbdee6f16c1cce6ull, 0xbc450f8e2fb71673ull, 0x3fefc7d078d1bc88ull, 0x3c8075d2447db685ull,           \
      0x3fbfeaaeee86ee36ull, 0xbc4afcb2bcc6f03bull, 0x3fefc015527d5bd3ull, 0x3c8b68f35094efb8ull,           \
      0x3fc0f3378ddd71d1ull, 0x3c6d8468724f0f9eull, 0x3fefb7db2bfe0695ull, 0x3c821dadf4f65ab1ull,           \
      0x3fc1f0d3d7afceafull, 0xbc66ef95099769a5ull, 0x3fefaf22263c4bd3ull, 0xbc552ace133a2769ull,           \
      0x3fc2ee285e4ab88full, 0xbc6e4d0f05dee058ull, 0x3fefa5ea641c36f2ull, 0x3c404da6ed17cc7cull,           \
      0x3fc3eb312c5d66cbull, 0x3c647d666b66cb91ull, 0x3fef9c340a7cc428ull, 0x3c8c5b6b063b7462ull,           \
      0x3fc4e7ea4dc5f27bull, 0x3c5949db2ac072fcull, 0x3fef91ff40374d01ull, 0xbc67d03f4d3a9e4cull,           \
      0x3fc5e44fcfa126f3ull, 0xbc66f443063f89b6ull, 0x3fef874c2e1eecf6ull, 0xbc8c6514e1332b16ull,           \
      0x3fc6e05dc05a4d4cull, 0xbbd32c5c8b81c919ull, 0x3fef7c1afeffde24ull, 0xbc78f55bc47540b1ull,           \
      0x3fc7dc102fbaf2b5ull, 0x3c45ab50e23c97c3ull, 0x3fef706bdf9ece1cull, 0xbc8698c80c36dcb4ull,           \
      0x3fc8d7632efaa944ull, 0xbc620fa262cbb953ull, 0x3fef643efeb82acdull, 0x3c76b00ac1fe28acull,           \
      0x3fc9d252d0cec312ull, 0x3c59c43d80b1137dull, 0x3fef57948cff6797ull, 0x3c6e3a0d3e03b1d4ull,           \
      0x3fcaccdb297a0765ull, 0xbc59883b57d6cdeaull, 0x3fef4a6cbd1e3a79ull, 0x3c813df0edaebb57ull,           \
      0x3fcbc6f84edc6199ull, 0x3c69c1a56a7b0cabull, 0x3fef3cc7c3b3d16eull, 0xbc621a3ad28a3494ull,           \
      0x3fccc0a6588289a3ull, 0xbc6868d09bc87c6bull, 0x3fef2ea5d753ffedull, 0x3c8cc4215f56d583ull,           \
      0x3fcdb9e15fb5a5d0ull, 0xbc632e20d6cc6fc2ull, 0x3fef20073086649full, 0x3c7b940416c1984bull,           \
      0x3fceb2a57f8ae5a3ull, 0xbc60be06af572cebull, 0x3fef10ec09c5873bull, 0x3c8d9072762c1283ull,           \
      0x3fcfaaeed4f31577ull, 0xbc615d88508e32b8ull, 0x3fef01549f7deea1ull, 0x3c8d3c1e99e5cafdull,           \
      0x3fd0515cbf65155cull, 0xbc79b8c29dfd8ec7ull, 0x3feef141300d2f26ull, 0xbc82aa1b08ded372ull,           \
      0x3fd0cd00cef36436ull, 0xbc79fb0a0c93e2b4ull, 0x3feee0b1fbc0f11cull, 0xbc4bfd2380bbc3b1ull,           \
      0x3fd14861aa94ddebull, 0xbc6be881b5b615a4ull, 0x3feecfa744d5efa1ull, 0xbc556d0a4af541d0ull,           \
      0x3fd1c37d64c6b876ull, 0x3c746076fe0dcff4ull, 0x3feebe214f76efa8ull, 0xbc802f9f12ba543eull,           \
      0x3fd23e52111aaf36ull, 0xbc74f080334eff18ull, 0x3feeac2061bbaf4full, 0x3c62c1d53e94658dull,           \
      0x3fd2b8ddc43eb49full, 0x3c61553899f2d807ull, 0x3fee99a4c3a7cd83ull, 0xbc82264b1bc53ce8ull,           \
      0x3fd3331e94049f87ull, 0x3c7e0cb6b40c302cull, 0x3fee86aebf29a9edull, 0x3c89397afdbb58a7ull,           \
      0x3fd3ad129769d3d8ull, 0x3c003d550487839aull, 0x3fee733ea0193d40ull, 0xbc86428b3546ce13ull,           \
      0x3fd426b7e69ee697ull, 0xbc7f09c75705c59full, 0x3fee5f54b436e9d0ull, 0x3c87eb0fd02fc8bcull,           \
      0x3fd4a00c9b0f3d20ull, 0x3c7823ba6bb08eadull, 0x3fee4af14b2a449cull, 0xbc868ca02e8a6833ull,           \
      0x3fd5190ecf68a77aull, 0x3c7b357155eef0f3ull, 0x3fee3614b680d6a5ull, 0xbc727793aa015237ull,           \
      0x3fd591bc9fa2f597ull, 0x3c67c74bac3fe0cbull, 0x3fee20bf49acd6c1ull, 0xbc5660aec7ef636bull,           \
      0x3fd60a1429078775ull, 0x3c5b1fd80ba89133ull, 0x3fee0af15a03dbceull, 0x3c5fe8e702771ae6ull,           \
      0x3fd682138a38d7f7ull, 0xbc7d889202444aadull, 0x3fedf4ab3ebd875eull, 0xbc8e2d8a7e6736c4ull,           \
      0x3fd6f9b8e33a0255ull, 0x3c742bc14ee9da0dull, 0x3feddded50f228d6ull, 0xbc6e80c8d42ba2bfull,           \
      0x3fd7710255764214ull, 0xbc66ead7314bb6ceull, 0x3fedc6b7eb995912ull, 0x3c54b364776dcd35ull,           \
      0x3fd7e7ee03c86d4eull, 0xbc7b63bcdabf5af2ull, 0x3fedaf0b6b888e83ull, 0x3c8a249e2b5e5ceaull,           \
      0x3fd85e7a12826949ull, 0x3c78a40e9b5face0ull, 0x3fed96e82f71a9dcull, 0x3c8ff61bd5d2039dull,           \
      0x3fd8d4a4a774992full, 0x3c744a02ea766326ull, 0x3fed7e4e97e17b4aull, 0xbc63b770352bed94ull,           \
      0x3fd94a6be9f546c5ull, 0xbc769ce13e683f58ull, 0x3fed653f073e4040ull, 0xbc876236434bec37ull,           \
      0x3fd9bfce02e80510ull, 0x3c709e39a320b0a4ull, 0x3fed4bb9e1c619e0ull, 0x3c8f34bb77858f61ull,           \
      0x3fda34c91cc50ccaull, 0xbc5a310e3b50cecdull, 0x3fed31bf8d8d7c06ull, 0x3c7e60dd3089cbddull,           \
      0x3fdaa95b63a09277ull, 0xbc66293eb13c0381ull, 0x3fed1750727d94f0ull, 0x3c80d52b1ec1a48eull,           \
      0x3fdb1d8305321617ull, 0xbc7ae242cb99f519ull, 0x3fecfc6cfa52ad9full, 0x3c88b5b5508f2a0dull,           \
      0x3fdb913e30dbac43ull, 0xbc7e38ad2f6c3ff1ull, 0x3fece115909a82e5ull, 0x3c81f139bb31109aull,           \
      0x3fdc048b17b140a3ull, 0x3c619fe6757e9fa7ull, 0x3fecc54aa2b2972eull, 0x3c64ee162ba83a98ull,           \
      0x3fdc7767ec7fd19eull, 0xbc5eb14d1a3d5826ull, 0x3feca90c9fc67d0bull, 0xbc646a81485e3462ull,           \
      0x3fdce9d2e3d4a51full, 0xbc62fc8a12dae298ull, 0x3fec8c5bf8ce1a84ull, 0x3c7ab3d1a1590123ull,           \
      0x3fdd5bca34047661ull, 0x3c728a44a75fc29cull, 0x3fec6f39208be53bull, 0xbc8741dbfbaadb42ull,           \
      0x3fddcd4c15329c9aull, 0x3c70d4c6e171fd9aull, 0x3fec51a48b8b175eull, 0xbc61bbb43b9aa880ull,           \
      0x3fde3e56c1582a69ull, 0xbc50a4821099f88full, 0x3fec339eb01ddd81ull, 0xbc8caaf5ee82c5c0ull,           \
      0x3fdeaee8744b05f0ull, 0xbc5789b43c9b027dull, 0x3fec1528065b7d50ull, 0xbc8892111312e828ull,           \
      0x3fdf1eff6bc4f97bull, 0x3c717212f8a7525cull, 0x3febf641081e7536ull, 0x3c8b7bd71628a9a1ull,           \
      0x3fdf8e99e76abc97ull, 0x3c59d950af2d00a3ull, 0x3febd6ea310294f5ull, 0x3c731bbcc88c109dull,           \
      0x3fdffdb628d2f57aull, 0x3c6f4a992e905b6aull, 0x3febb723fe630f32ull, 0x3c772bd2452d0a39ull,           \
      0x3fe0362939c69955ull, 0xbc82d8cd78397b01ull, 0x3feb96eeef58840eull, 0x3c545a3cc78fade0ull,           \
      0x3fe06d3686946e5bull, 0x3c83f5ae4538ff1bull, 0x3feb764b84b704c2ull, 0xbc8f5848c21b389bull,           \
      0x3fe0a4021e9e1001ull, 0xbc86f643a13914f6ull, 0x3feb553a410c104eull, 0x3c58ff7947027a15ull,           \
      0x3fe0da8b26b5672eull, 0xbc8a58def0bee909ull, 0x3feb33bba89c8948ull, 0x3c8ea6a51d1f6ca9ull,           \
      0x3fe110d0c4b69c3bull, 0x3c8d918998809981ull, 0x3feb11d04162a4c6ull, 0x3c71dd561efbc0c2ull,           \
      0x3fe146d21f8b7f82ull, 0x3c7bf9535e2739a8ull, 0x3feaef78930bd275ull, 0xbc7f836279746f94ull,           \
      0x3fe17c8e5f2eedb0ull, 0x3c635e57102e2488ull, 0x3feaccb526f69de5ull, 0x3c88fb6a8dd6b6ccull,           \
      0x3fe1b204acb02fddull, 0xbc5f190c70cbb5feull, 0x3feaa98688308913ull, 0xbc0b83d607cd5072ull,           \
      0x3fe1e7343236574cull, 0x3c722a3fa4f41d5aull, 0x3fea85ed4373e02dull, 0x3c69be06385ec792ull,           \
      0x3fe21c1c1b0394cfull, 0x3c5e5b324b23aa31ull, 0x3fea61e9e72586afull, 0x3c858330e2fd453full,           \
      0x3fe250bb93788bbbull, 0x3c7ea3d02457bcceull, 0x3fea3d7d0352bdcfull, 0xbc868dbaeca19669ull,           \
      0x3fe28511c917a067ull, 0xbc801df1d9a16b70ull, 0x3fea18a729aee445ull, 0x3c395e25736c0357ull,           \
      0x3fe2b91dea88421eull, 0xbc8fa371db216ab0ull, 0x3fe9f368ed912f85ull, 0xbc81d200c5791606ull,           \
      0x3fe2ecdf279a3082ull, 0x3c8d3557e0e7e37eull, 0x3fe9cdc2e3f25e5cull, 0x3c83f99112993f62ull,           \
      0x3fe32054b148bc4full, 0x3c8f6b42095a135bull, 0x3fe9a7b5a36a6514ull, 0x3c8722cfcc9fa7a9ull,           \
      0x3fe3537db9be0367ull, 0x3c6b327e7af040f0ull, 0x3fe98141c42e1310ull, 0x3c8d1ff80488f08dull,           \
      0x3fe386597456282bull, 0xbc710fada93b07a8ull, 0x3fe95a67e00cb1fdull, 0xbc80befda21f862dull,           \
      0x3fe3b8e715a2840aull, 0xbc797653a7d2f07aull, 0x3fe93328926d9e92ull, 0xbc8bb77003600cdaull,           \
      0x3fe3eb25d36cd53aull, 0xbc5be570e1570fc0ull, 0x3fe90b84784ddaf7ull, 0xbc70feb10ab93b87ull,           \
      0x3fe41d14e4ba6790ull, 0x3c84608fd287ecf5ull, 0x3fe8e37c303d9ad1ull, 0xbc6463a4b53d4bf8ull,           \
      0x3fe44eb381cf386bull, 0xbc83ed6c1e6a5505ull, 0x3fe8bb105a5dc900ull, 0x3c8863e03e9474c1ull,           \
      0x3fe48000e431159full, 0xbc8b194a7463ed10ull, 0x3fe89241985d871full, 0x3c8c48d9c413ed84ull,           \
      0x3fe4b0fc46aab761ull, 0x3c20da05738cc59cull, 0x3fe869108d77a6c6ull, 0x3c7338ffe2bfe9ddull,           \
      0x3fe4e1a4e54ed51bull, 0xbc8a492f89b7c76aull, 0x3fe83f7dde701ca0ull, 0xbc4152cf609bc6e8ull,           \
      0x3fe511f9fd7b351cull, 0xbc85c0e861c48831ull, 0x3fe8158a31916d5dull, 0xbc6de8b90b8228deull,           \
      0x3fe541facddbb724ull, 0x3c7232c28520d391ull, 0x3fe7eb362eaa1488ull, 0x3c5a1d65a4a5959full,           \
      0x3fe571a6966d59b3ull, 0x3c5c843b4d0fb197ull, 0x3fe7c0827f09e54full, 0xbc6c73d6d72aee68ull,           \
      0x3fe5a0fc98813a12ull, 0xbc8d82e2b7d4227bull, 0x3fe7956fcd7f6543ull, 0xbc8ab276e9d45ae4ull,           \
      0x3fe5cffc16bf8f0dull, 0x3c896cb370eb578aull, 0x3fe769fec655211full, 0xbc6827d5cf8c68c5ull,           \
      0x3fe5fea4552a9e57ull, 0x3c80b6cef7ee20b7ull, 0x3fe73e30174efba1ull, 0xbc65d3ae3d94ad5full,           \
      0x3fe62cf49921ac79ull, 0xbc8edd9855b6241aull, 0x3fe712046fa77678ull, 0x3c8425b0a5029c81ull,           \
      0x3fe65aec2963e755ull, 0x3c8126f96b71053cull, 0x3fe6e57c800cf55eull, 0x3c860286dedbd0a6ull,           \
      0x3fe6888a4e134b2full, 0xbc86b7d37644d5e6ull, 0x3fe6b898fa9efb5dull, 0x3c715ac786ccf4b2ull,           \
      0x3fe6b5ce50b7821aull, 0xbc65d5158f702e0full, 0x3fe68b5a92eb6253ull, 0xbc89a91ad985f89cull,           \
      0x3fe6e2b77c40bde1ull, 0xbc70e729857fad53ull, 0x3fe65dc1fdeb8cbaull, 0xbc597c1b47337c77ull,           \
      0x3fe70f451d0a8c40ull, 0x3c697ede3885770dull, 0x3fe62fcff20191c7ull, 0x3c6d9143895756efull,           \
      0x3fe73b7680dea578ull, 0xbc72248306dc12a2ull, 0x3fe6018526f563dfull, 0x3c846ca5e0e432d0ull,           \
      0x3fe7674af6f7b524ull, 0x3c7e9d3f94ac84a8ull, 0x3fe5d2e255f1f17aull, 0x3c80314104c8892bull,           \
      0x3fe792c1d0041d52ull, 0xbc8abf05eeb354ebull, 0x3fe5a3e839824077ull, 0x3c8428aa2759be62ull,           \
      0x3fe7bdda5e28b3c2ull, 0x3c4ad1197ccd0392ull, 0x3fe574978d8e83f2ull, 0x3c8f4714af282d23ull,           \
      0x3fe7e893f5037959ull, 0x3c80eefbaa650c4cull, 0x3fe544f10f592ca5ull, 0xbc8e7ae8e6c7a62full,           \
      0x3fe812ede9ae4ba4ull, 0xbc87830adf402ddaull, 0x3fe514f57d7bf3daull, 0x3c747a108073c259ull,           \
      0x3fe83ce792c1906eull, 0xbc7f3899682b4a7dull, 0x3fe4e4a597e4e10eull, 0x3c7ccd992849f6c8ull            \
    }
#define ZM_TOVERP_TAB                                                                                       \
    {                                                                                                       \
      10680707.0, 7228996.0, 1387004.0, 2578385.0, 16069853.0, 12639074.0, 9804092.0, 4427841.0,            \
      16666979.0, 11263675.0, 12935607.0, 2387514.0, 4345298.0, 14681673.0, 3074569.0, 13734428.0,          \
      16653803.0, 1880361.0, 10960616.0, 8533493.0, 3062596.0, 8710556.0, 7349940.0, 6258241.0,             \
      3772886.0, 3769171.0, 3798172.0, 8675211.0, 12450088.0, 3874808.0, 9961438.0, 366607.0,               \
      15675153.0, 9132554.0, 7151469.0, 3571407.0, 2607881.0, 12013382.0, 4155038.0, 6285869.0,             \
      7677882.0, 13102053.0, 15825725.0, 473591.0, 9065106.0, 15363067.0, 6271263.0, 9264392.0,             \
      5636912.0, 4652155.0, 7056368.0, 13614112.0, 10155062.0, 1944035.0, 9527646.0, 15080200.0,            \
      6658437.0, 6231200.0, 6832269.0, 16767104.0, 5075751.0, 3212806.0, 1398474.0, 7579849.0,              \
      6349435.0, 12618859.0, 4703257.0, 12806093.0, 14477321.0, 2786137.0, 12875403.0, 9837734.0,           \
      14528324.0, 13719321.0, 343717.0                                                                      \
    }
static const uint64_t kSinCos64TabHost[444] = ZM_SINCOS64_TAB;
static const double kToverpHost[75] = ZM_TOVERP_TAB;
#if defined(__HIPCC__)
static __device__ const uint64_t kSinCos64TabDev[444] = ZM_SINCOS64_TAB;
static __device__ const double kToverpDev[75] = ZM_TOVERP_TAB;
#endif
ZM_HD const double *sincos64_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return reinterpret_cast<const double *>(kSinCos64TabDev);
#else
    return reinterpret_cast<const double *>(kSinCos64TabHost);
#endif
}
ZM_HD const double *toverp_table()
{
#if defined(__HIP_DEVICE_COMPILE__)
    return kToverpDev;
#else
    return kToverpHost;
#endif
}

// the constants as data (a kernel argument: scalar registers feed the f64 operations directly)
struct SinCos64Coef {
    double big = 0x1.8p45, toint = 0x1.8p52, hpinv = 0x1.45f306dc9c883p-1;
    double hp0 = 0x1.921fb54442d18p0, hp1 = 0x1.1a62633145c07p-54;
    double mp1 = 0x1.921FB58000000p0, mp2 = -0x1.DDE973C000000p-27, pp3 = -0x1.CB3B398000000p-55, pp4 = -0x1.d747f23e32ed7p-83;
    double sn3 = -1.66666666666664880952546298448555E-01, sn5 = 8.33333214285722277379541354343671E-03;
    double cs2 = 4.99999999999999999999950396842453E-01, cs4 = -4.16666666666664434524222570944589E-02,
           cs6 = 1.38888874007937613028114285595617E-03;
    double s1 = -0x1.5555555555555p-3, s2 = 0x1.1111111110ECEp-7, s3 = -0x1.A01A019DB08B8p-13, s4 = 0x1.71DE27B9A7ED9p-19,
           s5 = -0x1.ADDFFC2FCDF59p-26;
};

// sin (n even) or cos (n odd) of a + da, negated for n = 2, 3 (the sources' do_sincos with do_sin, do_cos, TAYLOR_SIN).
// The two table paths are kept apart as in the sources: merged into one path with selected operands (both
// corrections read P s + (-M c + (s p + m)) for suitable M, m, P, p) the kernels measured 2 to 10 % slower.
ZM_HD double sincos64_eval(double a, double da, int n, const double *tab, const SinCos64Coef &k)
{
    const double aa = __builtin_fabs(a);
    double r;
    if ((n & 1) == 0 && aa < 0.126) {
        const double xx = a * a;
        double p = __builtin_fma(k.s5, xx, k.s4);
        p = __builtin_fma(p, xx, k.s3);
        p = __builtin_fma(p, xx, k.s2);
        p = __builtin_fma(p, xx, k.s1);
        const double t = __builtin_fma(__builtin_fma(p, a, -0.5 * da), xx, da);
        r = a + t;
    } else {
        const double u = k.big + aa;                     // its low mantissa bits: the nearest multiple of 1/128
        const double *e = tab + 4 * (int)(uint32_t)d2u(u);
        const double sn = e[0], ssn = e[1], cs = e[2], ccs = e[3];
        if (n & 1) {
            const double dx = a < 0 ? -da : da;
            const double x = aa - (u - k.big) + dx;
            const double xx = x * x;
            const double s = __builtin_fma(x * xx, __builtin_fma(xx, k.sn5, k.sn3), x);
            const double c = xx * __builtin_fma(xx, __builtin_fma(xx, k.cs6, k.cs4), k.cs2);
            const double cor = __builtin_fma(-sn, s, __builtin_fma(-cs, c, __builtin_fma(-s, ssn, ccs)));
            r = cs + cor;
        } else {
            const double dx = a <= 0 ? -da : da;
            const double x = aa - (u - k.big);
            const double xx = x * x;
            const double s = x + __builtin_fma(x * xx, __builtin_fma(xx, k.sn5, k.sn3), dx);
            const double c = __builtin_fma(x, dx, xx * __builtin_fma(xx, __builtin_fma(xx, k.cs6, k.cs4), k.cs2));
            const double cor = __builtin_fma(cs, s, __builtin_fma(-sn, c, __builtin_fma(s, ccs, ssn)));
            r = __builtin_copysign(sn + cor, a);
        }
    }
    return (n & 2) ? -r : r;
}

// |x| >= 105414350 (branred.c, then the evaluation above with quadrant n + nadd).  Out of line: few tensors hold
// such arguments.  (It builds its own constants: a reference to the caller's would force them into memory there.)
ZM_RARE double sincos64_huge(double x, int nadd, const double *tab)
{
    const SinCos64Coef k;
    const double tm600 = 0x1p-600, split = 134217729.0, tm24 = 0x1p-24, big = 0x1.8p52, big1 = 0x1.8p54;
    const double mp2 = -0x1.DDE9740000000p-27;           // branred.c's second piece of pi/2 is shorter than s_sin.c's
    const double *toverp = toverp_table();
    x *= tm600;
    double t = x * split;
    const double x1 = t - (t - x);
    const double x2 = x - x1;
    double b1 = 0, bb1 = 0, sum1 = 0, b2 = 0, bb2 = 0, sum2 = 0;
    for (int h = 0; h < 2; h++) {
        const double xp = h ? x2 : x1;
        double r[6], s, sum = 0;
        int j = (int)((d2u(xp) >> 52) & 2047u);
        j = (j - 450) / 24;
        if (j < 0) j = 0;
        double gor = u2d(d2u(0x1p576) - ((uint64_t)(j * 24) << 52));
        for (int i = 0; i < 6; i++) {
            r[i] = xp * toverp[j + i] * gor;
            gor *= tm24;
        }
        for (int i = 0; i < 3; i++) {
            s = (r[i] + big) - big;
            sum += s;
            r[i] -= s;
        }
        t = 0;
        for (int i = 0; i < 6; i++) t += r[5 - i];
        double bb = (((((r[0] - t) + r[1]) + r[2]) + r[3]) + r[4]) + r[5];
        s = (t + big) - big;
        sum += s;
        t -= s;
        const double b = t + bb;
        bb = (t - b) + bb;
        s = (sum + big1) - big1;
        sum -= s;
        if (h) { b2 = b; bb2 = bb; sum2 = sum; }
        else { b1 = b; bb1 = bb; sum1 = sum; }
    }
    double sum = sum1 + sum2;
    double b = b1 + b2;
    double bb = (__builtin_fabs(b1) > __builtin_fabs(b2)) ? (b1 - b) + b2 : (b2 - b) + b1;
    if (b > 0.5) { b -= 1.0; sum += 1.0; }
    else if (b < -0.5) { b += 1.0; sum -= 1.0; }
    double s = b + (bb + bb1 + bb2);
    t = ((b - s) + bb) + (bb1 + bb2);
    b = s * split;
    const double t1 = b - (b - s);
    const double t2 = s - t1;
    b = s * k.hp0;
    bb = (((t1 * k.mp1 - b) + t1 * mp2) + t2 * k.mp1) + (t2 * mp2 + s * k.hp1 + t * k.hp0);
    s = b + bb;
    t = (b - s) + bb;
    return sincos64_eval(s, t, (int)sum + nadd, tab, k);
}

// x - n pi/2 for |x| < 105414350 as a + da; returns n + nadd
ZM_HD int sincos64_reduce(double x, int nadd, double &a, double &da, const SinCos64Coef &k)
{
    const double t = __builtin_fma(x, k.hpinv, k.toint);
    const double xn = t - k.toint;
    const double y = __builtin_fma(-xn, k.mp2, __builtin_fma(-xn, k.mp1, x));
    double t1 = xn * k.pp3;
    const double t2 = y - t1;
    double db = (y - t2) - t1;
    t1 = xn * k.pp4;
    const double b = t2 - t1;
    db += (t2 - b) - t1;
    a = b;
    da = db;
    return (int)(uint32_t)d2u(t) + nadd;
}

ZM_HD double sin_glibc(double x, const double *tab, const SinCos64Coef &k = SinCos64Coef())
{
    const uint32_t hi = (uint32_t)(d2u(x) >> 32) & 0x7fffffffu;
    if (hi < 0x3e500000u) return x;                      // |x| < 2^-26
    double a, da;
    int n;
    if (hi < 0x3feb6000u) {                              // |x| < 0.855469
        a = x;
        da = 0.0;
        n = 0;
    } else if (hi < 0x400368fdu) {                       // |x| < 2.426265: cos(pi/2 - |x|) with the sign of x
        a = k.hp0 - __builtin_fabs(x);
        da = k.hp1;
        n = (d2u(x) >> 63) ? 3 : 1;
    } else if (hi < 0x419921FBu) {                       // |x| < 105414350
        n = sincos64_reduce(x, 0, a, da, k);
    } else if (hi < 0x7ff00000u) {
        return sincos64_huge(x, 0, tab);
    } else {
        return x - x;                                    // inf, NaN (the sources' x / x)
    }
    return sincos64_eval(a, da, n, tab, k);
}

ZM_HD double cos_glibc(double x, const double *tab, const SinCos64Coef &k = SinCos64Coef())
{
    const uint32_t hi = (uint32_t)(d2u(x) >> 32) & 0x7fffffffu;
    if (hi < 0x3e400000u) return 1.0;                    // |x| < 2^-27
    double a, da;
    int n;
    if (hi < 0x3feb6000u) {
        a = x;
        da = 0.0;
        n = 1;
    } else if (hi < 0x400368fdu) {                       // sin(pi/2 - |x|), the difference renormalised
        const double y = k.hp0 - __builtin_fabs(x);
        a = y + k.hp1;
        da = (y - a) + k.hp1;
        n = 0;
    } else if (hi < 0x419921FBu) {
        n = sincos64_reduce(x, 1, a, da, k);
    } else if (hi < 0x7ff00000u) {
        return sincos64_huge(x, 1, tab);
    } else {
        return x - x;
    }
    return sincos64_eval(a, da, n, tab, k);
}
ZM_HD double sin_glibc(double x) { return sin_glibc(x, sincos64_table()); }
ZM_HD double cos_glibc(double x) { return cos_glibc(x, sincos64_table()); }

#if defined(__HIPCC__)
// exp / log / sinh / cosh as the kernels call them: through tables copied to LDS by init(), which
// every thread of the workgroup (at least 64 threads) calls once before anything else (it
// synchronises).
template <typename T> struct ExpLog;
template <> struct ExpLog<double> {
    const uint64_t *etab;
    ExpCoef64 ek;
    Expm1Coef64 mk;
    const double *ltab;
    LogCoef64 lk;
    __device__ __forceinline__ void init(bool need_exp, bool need_log)
    {
        __shared__ uint64_t lds_exp64[256];
        __shared__ uint64_t lds_log64[256];
        if (threadIdx.x < 64) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                if (need_exp) lds_exp64[threadIdx.x + 64 * i] = kExpTabDev[threadIdx.x + 64 * i];
                if (need_log) lds_log64[threadIdx.x + 64 * i] = kLog64TabDev[threadIdx.x + 64 * i];
            }
        }
        __syncthreads();
        etab = lds_exp64;
        ltab = reinterpret_cast<const double *>(lds_log64);
    }
    __device__ __forceinline__ double exp(double x) const { return exp_glibc(x, etab, ek); }
    __device__ __forceinline__ double exp_flat(double x) const { return exp_glibc(x, etab, ek); }
    __device__ __forceinline__ double log(double x) const { return log_glibc(x, ltab, lk); }
    __device__ __forceinline__ double sinh(double x) const { return sinh_simd(x, etab, mk); }
    __device__ __forceinline__ double cosh(double x) const { return cosh_simd(x, etab, mk, ek); }
    __device__ __forceinline__ double sinh(double x, const TanhRegs &) const { return sinh_simd(x, etab, mk); }
    __device__ __forceinline__ double cosh(double x, const TanhRegs &) const { return cosh_simd(x, etab, mk, ek); }
    // no table: usable without init()
    __device__ __forceinline__ double tanh(double x, const TanhRegs &) const { return tanh_simd(x, mk); }
    __device__ __forceinline__ double sigmoid(double x, const TanhRegs &) const { return sigmoid_zenu(x, mk); }
};
template <> struct ExpLog<float> {
    const uint64_t *etab;
    const double *ltab;
    __device__ __forceinline__ void init(bool need_exp, bool need_log)
    {
        __shared__ uint64_t lds_exp[32];
        __shared__ double lds_log[32];
        if (threadIdx.x < 32) {
            if (need_exp) lds_exp[threadIdx.x] = kExp2fTabDev[threadIdx.x];
            if (need_log) lds_log[threadIdx.x] = kLogfTabDev[threadIdx.x];
        }
        __syncthreads();
        etab = lds_exp;
        ltab = lds_log;
    }
    ExpfCoef ek;
    LogfCoef lk;
    __device__ __forceinline__ float exp(float x) const { return expf_glibc(x, etab, ek); }
    __device__ __forceinline__ float exp_flat(float x) const { return expf_glibc_flat(x, etab, ek); }
    __device__ __forceinline__ float log(float x) const { return logf_glibc(x, ltab, lk); }
    __device__ __forceinline__ float sinh(float x) const { return sinhf_simd(x, etab); }
    __device__ __forceinline__ float cosh(float x) const { return coshf_simd(x, etab, TanhRegs(), ek); }
    // with the two register-held constants of the expm1 core pinned by the caller
    __device__ __forceinline__ float sinh(float x, const TanhRegs &rg) const { return sinhf_simd(x, etab, rg); }
    __device__ __forceinline__ float cosh(float x, const TanhRegs &rg) const { return coshf_simd(x, etab, rg, ek); }
    // no table: usable without init()
    __device__ __forceinline__ float tanh(float x, const TanhRegs &rg) const { return tanhf_simd(x, rg); }
    __device__ __forceinline__ float sigmoid(float x, const TanhRegs &rg) const { return sigmoidf_zenu(x, rg); }
};

// atanf's range table in LDS, same arrangement (init() by every thread of the workgroup, once)
struct AtanfLds {
    const float *tab;
    __device__ __forceinline__ void init()
    {
        __shared__ float lds_atan[40];
        if (threadIdx.x < 40) lds_atan[threadIdx.x] = kAtanfTabDev[threadIdx.x];
        __syncthreads();
        tab = lds_atan;
    }
};

// the f64 sine / cosine table in LDS, same arrangement
struct SinCos64Lds {
    const double *tab;
    __device__ __forceinline__ void init()
    {
        __shared__ uint64_t lds_sincos[444];
        for (int i = threadIdx.x; i < 444; i += blockDim.x) lds_sincos[i] = kSinCos64TabDev[i];
        __syncthreads();
        tab = reinterpret_cast<const double *>(lds_sincos);
    }
};

// pow with the same arrangement: its log and exp tables in LDS
template <typename T> struct Pow;
template <> struct Pow<double> {
    const double *ltab;
    const uint64_t *etab;
    __device__ __forceinline__ void init()
    {
        __shared__ uint64_t lds_powlog[384];
        __shared__ uint64_t lds_powexp[256];
        for (int i = threadIdx.x; i < 384; i += blockDim.x) lds_powlog[i] = kPow64LogTabDev[i];
        for (int i = threadIdx.x; i < 256; i += blockDim.x) lds_powexp[i] = kExpTabDev[i];
        __syncthreads();
        ltab = reinterpret_cast<const double *>(lds_powlog);
        etab = lds_powexp;
    }
    PowCoef64 k;
    __device__ __forceinline__ double pow(double x, double y) const { return pow_glibc(x, y, ltab, etab, k); }
};
template <> struct Pow<float> {
    const uint64_t *etab;
    const double *ltab;
    __device__ __forceinline__ void init()
    {
        __shared__ uint64_t lds_exp2[32];
        __shared__ double lds_log2[32];
        if (threadIdx.x < 32) {
            lds_exp2[threadIdx.x] = kExp2fTabDev[threadIdx.x];
            lds_log2[threadIdx.x] = kPowfLog2TabDev[threadIdx.x];
        }
        __syncthreads();
        etab = lds_exp2;
        ltab = lds_log2;
    }
    PowCoef k;
    __device__ __forceinline__ float pow(float x, float y) const { return powf_glibc(x, y, etab, ltab, k); }
};
#endif

}  // namespace ZMATH_NS

#undef ZMATH_EMIT
#undef ZMATH_NS
#endif  // ZMATH_EMIT
