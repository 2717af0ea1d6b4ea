// Host build of zenu_amd/csrc/zmath.hpp compared with the host libm (the functions ZeNu's CPU path
// calls through Rust's f32::tanh / exp / ln and f64::tanh).  Usage: zmath_host_check <stride>; checks every stride-th f32
// bit pattern (stride 1 = exhaustive, about ten minutes on 8 cores).  powf: every stride-th x for a set
// of fixed exponents, and 2^32 / stride pseudo-random (x, y) pairs.  Prints the mismatch counts.
#include <atomic>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <thread>
#include <vector>

#include "../../zenu_amd/csrc/zmath.hpp"

// sin and cos through pointers the compiler cannot see through: called on the same argument side by side
// they would be merged into one sincos call, which is another function of the library (it reduces
// |x| < 2.426265 differently and differs from sin / cos in the last bit on 1 in 1000 of such arguments)
static double (*volatile libm_sin)(double) = sin;
static double (*volatile libm_cos)(double) = cos;

int main(int argc, char **argv)
{
    const uint64_t stride = argc > 1 ? strtoull(argv[1], nullptr, 10) : 1;
    const int nt = 8;
    std::atomic<uint64_t> bad_fdlibm{0}, bad_simd{0}, bad_expm1{0}, bad_sig{0}, bad_exp{0}, bad_log{0}, bad_sinh{0}, bad_cosh{0}, bad_sin{0}, bad_cos{0}, bad_atan{0}, bad_asin{0}, bad_acos{0}, far_ulp2{0}, bad_sinh_simd{0}, bad_cosh_simd{0}, bad_tan{0};
    std::vector<std::thread> th;
    for (int w = 0; w < nt; w++)
        th.emplace_back([&, w]() {
            uint64_t b0 = 0, b1 = 0, b2 = 0, b3 = 0, b4 = 0, b5 = 0, b6 = 0, b7 = 0, b8 = 0, b9 = 0, b10 = 0, b11 = 0, b12 = 0, b13 = 0, b14 = 0, b15 = 0, b16 = 0;
            for (uint64_t u = (uint64_t)w * stride; u < (1ull << 32); u += stride * nt) {
                const float x = zmath::u2f((uint32_t)u);
                const float atr = atanf(x), atg = zmath::atanf_fdlibm(x);
                if ((atr != atr) ? !(atg != atg) : zmath::f2u(atg) != zmath::f2u(atr)) b10++;
                const float asr = asinf(x), asg = zmath::asinf_fdlibm(x);
                if ((asr != asr) ? !(asg != asg) : zmath::f2u(asg) != zmath::f2u(asr)) b11++;
                const float acr = acosf(x), acg = zmath::acosf_fdlibm(x);
                if ((acr != acr) ? !(acg != acg) : zmath::f2u(acg) != zmath::f2u(acr)) b12++;
                const float tnr = tanf(x), tng = zmath::tanf_glibc(x);
                if ((tnr != tnr) ? !(tng != tng) : zmath::f2u(tng) != zmath::f2u(tnr)) b16++;
                const float snr = sinf(x), sng = zmath::sinf_glibc(x);
                if ((snr != snr) ? !(sng != sng) : zmath::f2u(sng) != zmath::f2u(snr)) b8++;
                const float csr = cosf(x), csg = zmath::cosf_glibc(x);
                if ((csr != csr) ? !(csg != csg) : zmath::f2u(csg) != zmath::f2u(csr)) b9++;
                const float shr = sinhf(x), shg = zmath::sinhf_fdlibm(x);
                if ((shr != shr) ? !(shg != shg) : zmath::f2u(shg) != zmath::f2u(shr)) b6++;
                const float shs = zmath::sinhf_simd(x, zmath::exp2f_table());
                if ((shr != shr) ? !(shs != shs) : zmath::f2u(shs) != zmath::f2u(shr)) b14++;
                const float chr = coshf(x), chg = zmath::coshf_fdlibm(x);
                if ((chr != chr) ? !(chg != chg) : zmath::f2u(chg) != zmath::f2u(chr)) b7++;
                const float chs = zmath::coshf_simd(x, zmath::exp2f_table());
                if ((chr != chr) ? !(chs != chs) : zmath::f2u(chs) != zmath::f2u(chr)) b15++;
                const float er = expf(x), eg = zmath::expf_glibc(x);
                if ((er != er) ? !(eg != eg) : zmath::f2u(eg) != zmath::f2u(er)) b4++;
                const float lr = logf(x), lg = zmath::logf_glibc(x);
                if ((lr != lr) ? !(lg != lg) : zmath::f2u(lg) != zmath::f2u(lr)) b5++;
                const float ref = tanhf(x);
                const float a = zmath::tanhf_fdlibm(x), s = zmath::tanhf_simd(x);
                const bool nan = ref != ref;
                if (nan ? !(a != a) : zmath::f2u(a) != zmath::f2u(ref)) b0++;
                if (nan ? !(s != s) : zmath::f2u(s) != zmath::f2u(ref)) b1++;
                // the variant that is allowed 2 units in the last place: count what is further away
                const float q = zmath::tanhf_ulp2(x);
                if (nan ? !(q != q)
                        : ((q < 0) != (ref < 0) && q != ref) ||
                              (zmath::f2u(q) > zmath::f2u(ref) ? zmath::f2u(q) - zmath::f2u(ref) : zmath::f2u(ref) - zmath::f2u(q)) > 2)
                    b13++;
                if (fabsf(x) < 44.0f && zmath::f2u(zmath::expm1f_fdlibm(x)) != zmath::f2u(expm1f(x))) b2++;
                const float sg = 0.5f + 0.5f * tanhf(0.5f * x), sz = zmath::sigmoidf_zenu(x);
                if ((sg != sg) ? !(sz != sz) : zmath::f2u(sz) != zmath::f2u(sg)) b3++;
            }
            bad_fdlibm += b0; bad_simd += b1; bad_expm1 += b2; bad_sig += b3; bad_exp += b4; bad_log += b5; bad_sinh += b6; bad_cosh += b7; bad_sin += b8; bad_cos += b9; bad_atan += b10; bad_asin += b11; bad_acos += b12; far_ulp2 += b13; bad_sinh_simd += b14; bad_cosh_simd += b15; bad_tan += b16;
        });
    for (auto &t : th) t.join();
    // double precision: every stride-th value of the HIGH word (sign, exponent, 20 mantissa bits) with
    // a pseudo-random low word, plus low words 0 and all-ones
    std::atomic<uint64_t> bad_tanh64{0}, bad_expm164{0}, bad_sig64{0}, bad_exp64{0}, bad_sinh64{0}, bad_cosh64{0}, bad_sin64{0}, bad_cos64{0}, bad_log64{0};
    th.clear();
    for (int w = 0; w < nt; w++)
        th.emplace_back([&, w]() {
            uint64_t b0 = 0, b1 = 0, b2 = 0, b3 = 0, b4 = 0, b5 = 0, b6 = 0, b7 = 0, b8 = 0, rng = 0x9E3779B97F4A7C15ull * (w + 1);
            uint64_t round = 0;
            for (uint64_t u = (uint64_t)w * stride; u < (1ull << 32); u += stride * nt) {
                rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
                const uint32_t lows[3] = {(uint32_t)rng, 0u, 0xffffffffu};
                const bool trig = (round++ & 7) == 0;     // sin / cos on every eighth high word (the host libm takes 100 ns on large arguments)
                for (uint32_t lo : lows) {
                    const double x = zmath::u2d((u << 32) | lo);
                    const double ref = tanh(x), got = zmath::tanh_fdlibm(x), got2 = zmath::tanh_simd(x);
                    if ((ref != ref) ? !(got != got) : zmath::d2u(got) != zmath::d2u(ref)) b0++;
                    if ((ref != ref) ? !(got2 != got2) : zmath::d2u(got2) != zmath::d2u(ref)) b0++;   // the form the kernels use
                    if (fabs(x) < 700.0 && zmath::d2u(zmath::expm1_fdlibm(x)) != zmath::d2u(expm1(x))) b1++;
                    const double sg = 0.5 + 0.5 * tanh(0.5 * x), sz = zmath::sigmoid_zenu(x);
                    if ((sg != sg) ? !(sz != sz) : zmath::d2u(sz) != zmath::d2u(sg)) b2++;
                    const double er = exp(x), eg = zmath::exp_glibc(x);
                    if ((er != er) ? !(eg != eg) : zmath::d2u(eg) != zmath::d2u(er)) b3++;
                    const double shr = sinh(x), shg = zmath::sinh_fdlibm(x), shs = zmath::sinh_simd(x, zmath::exp_table());
                    if ((shr != shr) ? !(shg != shg) : zmath::d2u(shg) != zmath::d2u(shr)) b4++;
                    if ((shr != shr) ? !(shs != shs) : zmath::d2u(shs) != zmath::d2u(shr)) b4++;   // the form the kernels use
                    const double chr = cosh(x), chg = zmath::cosh_fdlibm(x), chs = zmath::cosh_simd(x, zmath::exp_table());
                    if ((chr != chr) ? !(chg != chg) : zmath::d2u(chg) != zmath::d2u(chr)) b5++;
                    if ((chr != chr) ? !(chs != chs) : zmath::d2u(chs) != zmath::d2u(chr)) b5++;   // the form the kernels use
                    const double lgr = log(x), lgg = zmath::log_glibc(x);
                    if ((lgr != lgr) ? !(lgg != lgg) : zmath::d2u(lgg) != zmath::d2u(lgr)) b8++;
                    if (trig) {
                        const double snr = libm_sin(x), sng = zmath::sin_glibc(x), csr = libm_cos(x), csg = zmath::cos_glibc(x);
                        if ((snr != snr) ? !(sng != sng) : zmath::d2u(sng) != zmath::d2u(snr)) b6++;
                        if ((csr != csr) ? !(csg != csg) : zmath::d2u(csg) != zmath::d2u(csr)) b7++;
                    }
                }
                // arguments where exp is finite and not 1: uniform in +-745 and in +-4
                const double m = (double)(int64_t)rng / 9.2233720368547758e18;
                // tanh and the sigmoid where they are neither x nor +-1: uniform in +-1, +-4 and +-20
                for (double x : {m, m * 4.0, m * 20.0}) {
                    if (zmath::d2u(zmath::sinh_simd(x, zmath::exp_table())) != zmath::d2u(sinh(x))) b4++;
                    if (zmath::d2u(zmath::cosh_simd(x, zmath::exp_table())) != zmath::d2u(cosh(x))) b5++;
                    const double ref = tanh(x);
                    if (zmath::d2u(zmath::tanh_fdlibm(x)) != zmath::d2u(ref) || zmath::d2u(zmath::tanh_simd(x)) != zmath::d2u(ref)) b0++;
                    if (zmath::d2u(zmath::sigmoid_zenu(x)) != zmath::d2u(0.5 + 0.5 * tanh(0.5 * x))) b2++;
                }
                // sin / cos in each of their argument ranges: +-0.855, +-2.43, +-10, +-1000, +-1e6, +-1.05e8
                if (trig)
                    for (double x : {m * 0.855, m * 2.43, m * 10.0, m * 1000.0, m * 1e6, m * 1.05e8}) {
                        if (zmath::d2u(zmath::sin_glibc(x)) != zmath::d2u(libm_sin(x))) b6++;
                        if (zmath::d2u(zmath::cos_glibc(x)) != zmath::d2u(libm_cos(x))) b7++;
                    }
                // log around 1 (both of its branches), on [0, 100) and log-uniform over the whole range
                for (double x : {1.0 + m * 0.5, fabs(m) * 100.0, exp(m * 700.0)})
                    if (zmath::d2u(zmath::log_glibc(x)) != zmath::d2u(log(x))) b8++;
                for (double x : {m * 745.0, m * 4.0}) {
                    const double er = exp(x), eg = zmath::exp_glibc(x);
                    if (zmath::d2u(eg) != zmath::d2u(er)) b3++;
                    const double shr = sinh(x), shg = zmath::sinh_fdlibm(x);
                    if (zmath::d2u(shg) != zmath::d2u(shr)) b4++;
                    const double chr = cosh(x), chg = zmath::cosh_fdlibm(x);
                    if (zmath::d2u(chg) != zmath::d2u(chr)) b5++;
                }
            }
            bad_tanh64 += b0; bad_expm164 += b1; bad_sig64 += b2; bad_exp64 += b3; bad_sinh64 += b4; bad_cosh64 += b5; bad_sin64 += b6; bad_cos64 += b7; bad_log64 += b8;
        });
    for (auto &t : th) t.join();
    // pow(x, y) in double: both forms (the complete routine and the one the kernels inline) on uniform bit patterns
    // for both arguments, on moderate pairs, and on negative / log-uniform bases under fixed exponents
    std::atomic<uint64_t> bad_pow64{0};
    th.clear();
    for (int w = 0; w < nt; w++)
        th.emplace_back([&, w]() {
            uint64_t b = 0, rng = 0xA0761D6478BD642Full * (w + 1);
            auto next = [&]() { rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17; return rng; };
            auto one = [&](double x, double y) {
                const double ref = pow(x, y), got = zmath::pow_glibc_full(x, y), got2 = zmath::pow_glibc(x, y);
                if ((ref != ref) ? !(got != got) : zmath::d2u(got) != zmath::d2u(ref)) b++;
                if ((ref != ref) ? !(got2 != got2) : zmath::d2u(got2) != zmath::d2u(ref)) b++;
            };
            const double ys[] = {2.0, 0.5, 2.5, -1.0, 3.0, -0.5, 1.0 / 3.0, 0.0, 1.0, -2.0, 10.25, 1e-3, 55.0, -3.0, 1e-20, 1e300,
                                 INFINITY, -INFINITY, NAN, 0x1p-66, 0x1p63, 4503599627370497.0};
            for (uint64_t u = (uint64_t)w * stride * 16; u < (1ull << 32); u += stride * nt * 16) {
                one(zmath::u2d(next()), zmath::u2d(next()));
                const double m1 = (double)(next() >> 11) * 0x1p-53, m2 = (double)(int64_t)next() / 9.2233720368547758e18;
                one(m1 * 4.0, m2 * 40.0);
                one(0.5 + m1, m2 * 1000.0);
                one(exp(m2 * 300.0), ys[next() % 22]);
                one(m2 * 10.0, ys[next() % 22]);
                one(zmath::u2d(next()), ys[next() % 22]);
            }
            bad_pow64 += b;
        });
    for (auto &t : th) t.join();
    // powf(x, y)
    std::atomic<uint64_t> bad_pow{0};
    th.clear();
    for (int w = 0; w < nt; w++)
        th.emplace_back([&, w]() {
            uint64_t b = 0, rng = 0xD1B54A32D192ED03ull * (w + 1);
            auto one = [&](float x, float y) {
                const float ref = powf(x, y), got = zmath::powf_glibc(x, y);
                if ((ref != ref) ? !(got != got) : zmath::f2u(got) != zmath::f2u(ref)) b++;
            };
            const float ys[] = {2.0f, 0.5f, 2.5f, -1.0f, 3.0f, 1.5f, -0.5f, 0.333333343f, 10.0f, -2.5f, 0.0f, 1.0f,
                                INFINITY, -INFINITY, NAN, zmath::u2f(0x7f800001u), 1e-30f, 16777217.0f, 5.0f};
            for (uint64_t u = (uint64_t)w * stride; u < (1ull << 32); u += stride * nt) {
                for (float y : ys) one(zmath::u2f((uint32_t)u), y);
                rng ^= rng << 13; rng ^= rng >> 7; rng ^= rng << 17;
                one(zmath::u2f((uint32_t)rng), zmath::u2f((uint32_t)(rng >> 32)));
                // moderate arguments, where the result is finite and the tables decide it
                const float xm = zmath::u2f(0x3c000000u + (uint32_t)(rng % 0x08000000u));           // [2^-7, 2^9)
                const float ym = zmath::u2f((0x3c000000u + (uint32_t)((rng >> 29) % 0x07000000u)) | ((uint32_t)(rng >> 63) << 31));
                one(xm, ym);
            }
            bad_pow += b;
        });
    for (auto &t : th) t.join();
    printf("tanhf_fdlibm %llu tanhf_simd %llu expm1f_fdlibm %llu sigmoidf_zenu %llu\n",
           (unsigned long long)bad_fdlibm.load(), (unsigned long long)bad_simd.load(),
           (unsigned long long)bad_expm1.load(), (unsigned long long)bad_sig.load());
    printf("tanh_fdlibm %llu expm1_fdlibm %llu sigmoid_zenu %llu\n", (unsigned long long)bad_tanh64.load(),
           (unsigned long long)bad_expm164.load(), (unsigned long long)bad_sig64.load());
    printf("exp_glibc %llu sinh_fdlibm %llu cosh_fdlibm %llu\n", (unsigned long long)bad_exp64.load(),
           (unsigned long long)bad_sinh64.load(), (unsigned long long)bad_cosh64.load());
    printf("expf_glibc %llu logf_glibc %llu\n", (unsigned long long)bad_exp.load(), (unsigned long long)bad_log.load());
    printf("powf_glibc %llu sinhf_fdlibm %llu coshf_fdlibm %llu\n", (unsigned long long)bad_pow.load(),
           (unsigned long long)bad_sinh.load(), (unsigned long long)bad_cosh.load());
    printf("sinhf_simd %llu coshf_simd %llu\n", (unsigned long long)bad_sinh_simd.load(), (unsigned long long)bad_cosh_simd.load());
    printf("sinf_glibc %llu cosf_glibc %llu\n", (unsigned long long)bad_sin.load(), (unsigned long long)bad_cos.load());
    printf("atanf_fdlibm %llu asinf_fdlibm %llu acosf_fdlibm %llu\n", (unsigned long long)bad_atan.load(),
           (unsigned long long)bad_asin.load(), (unsigned long long)bad_acos.load());
    printf("tanhf_ulp2_beyond_2ulp %llu tanf_glibc %llu\n", (unsigned long long)far_ulp2.load(), (unsigned long long)bad_tan.load());
    printf("sin_glibc %llu cos_glibc %llu log_glibc %llu\n", (unsigned long long)bad_sin64.load(), (unsigned long long)bad_cos64.load(), (unsigned long long)bad_log64.load());
    printf("pow_glibc %llu\n", (unsigned long long)bad_pow64.load());
    return (bad_pow64 + bad_log64 + bad_sin64 + bad_cos64 + bad_tan + bad_sinh_simd + bad_cosh_simd + far_ulp2 + bad_fdlibm + bad_simd + bad_expm1 + bad_sig + bad_tanh64 + bad_expm164 + bad_sig64 + bad_exp64 + bad_sinh64 + bad_cosh64 + bad_exp + bad_log + bad_pow + bad_sinh + bad_cosh + bad_sin + bad_cos + bad_atan + bad_asin + bad_acos) ? 1 : 0;
}
