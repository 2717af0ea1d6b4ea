// Rebuilds the {invc, logc} table of glibc's double-precision log (ZM_LOG64_TAB in ../zmath.hpp).
//
// The table is not defined by a formula.  Its authors (ARM's optimized routines, log_data.c) describe the
// construction: for each of the 128 subintervals of [0.6875, 1.375), try the 2^30 doubles around 1 / centre
// as invc and keep one for which log(c), c = 1 / invc, is within 2^-66 of a multiple of 2^-43 (so that
// logc = (double)log(c) has its low bits clear and k ln2_hi + logc is exact), subject to further conditions
// that only matter to the build without fused multiply-add.  This program lists every invc of that range
// that meets the first condition (about 420 per subinterval) and lets the host libm decide: the entry is
// the candidate with which the routine returns libm's bits on 10^5 random arguments of the subinterval
// scaled by several powers of two.  For every subinterval exactly one candidate survives; the full
// routine with the resulting table is then compared on 8e8 arguments (tests/native/zmath_host_check.cpp
// keeps a part of that).
//
//   g++ -O2 -std=gnu++17 -fext-numeric-literals -ffp-contract=off -mfma -fopenmp log64_table.cpp -lquadmath
//   ./a.out > table.txt        (three minutes on eight cores; "./a.out first last" does subintervals first .. last - 1)
#include <quadmath.h>
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

static inline uint64_t d2u(double f) { uint64_t u; memcpy(&u, &f, 8); return u; }
static inline double u2d(uint64_t u) { double f; memcpy(&f, &u, 8); return f; }

// the routine's main path (the constants are the sources'; every a + b c fused, as in the x86-64 FMA build)
static const double A[] = {-0x1.0000000000001p-1, 0x1.555555551305bp-2, -0x1.fffffffeb459p-3, 0x1.999b324f10111p-3, -0x1.55575e506c89fp-3};
static const double Ln2hi = 0x1.62e42fefa3800p-1, Ln2lo = 0x1.ef35793c76730p-45;
static double log_main(double x, double invc, double logc)
{
    const uint64_t ix = d2u(x);
    const uint64_t tmp = ix - 0x3fe6000000000000ull;
    const int64_t k = (int64_t)tmp >> 52;
    const double z = u2d(ix - (tmp & (0xfffull << 52)));
    const double r = __builtin_fma(z, invc, -1.0);
    const double kd = (double)k;
    const double w = __builtin_fma(kd, Ln2hi, logc);
    const double hi = w + r;
    const double lo = __builtin_fma(kd, Ln2lo, (w - hi) + r);
    const double r2 = r * r;
    const double p = __builtin_fma(r2, __builtin_fma(r, A[4], A[3]), __builtin_fma(r, A[2], A[1]));
    double y = __builtin_fma(r2, A[0], lo);
    y = __builtin_fma(r * r2, p, y);
    return y + hi;
}

struct Entry { double invc, logc; };

int main(int argc, char **argv)
{
    const int first = argc > 2 ? atoi(argv[1]) : 0, last = argc > 2 ? atoi(argv[2]) : 128;
    std::vector<Entry> table(128);
    std::vector<int> survivors(128);
#pragma omp parallel for schedule(dynamic)
    for (int i = first; i < last; i++) {
        const double lo = i < 80 ? 0.6875 + i / 256.0 : 1.0 + (i - 80) / 128.0;
        const double width = i < 80 ? 1 / 256.0 : 1 / 128.0;
        const double invc0 = 1.0 / (lo + width / 2);
        const double ulp = u2d(d2u(invc0) + 1) - invc0;
        // log(c) in units of 2^-43, modulo 1: exactly for the centre, by its series for the neighbours
        const __float128 L0 = -logq((__float128)invc0) * 0x1p43Q;
        const long double f0 = (long double)(L0 - floorq(L0));
        const long double tu = (long double)ulp / (long double)invc0;
        std::vector<Entry> cand;
        for (int64_t j = -(1ll << 29); j <= (1ll << 29); j++) {
            const long double t = tu * (long double)j;
            const long double s = (t - t * t * 0.5L + t * t * t * (1.0L / 3.0L)) * 0x1p43L;
            long double f = f0 - s;
            f -= floorl(f);
            const long double d = f > 0.5L ? 1.0L - f : f;
            if (d < 0x1p-23L) {                                  // 2^-66 in units of 2^-43
                const double invc = u2d(d2u(invc0) + j);
                const __float128 L = -logq((__float128)invc) * 0x1p43Q;
                cand.push_back({invc, (double)(roundq(L) * 0x1p-43Q)});
            }
        }
        std::mt19937_64 g(9 + i);
        for (int round = 0; round < 400 && cand.size() > 1; round++) {
            std::vector<double> xs, ref;
            for (int s = 0; s < 100000; s++) {
                static const int ks[] = {0, 1, -1, 7, -30, 500, 2, -2};
                const double x = ldexp(lo + width * ((double)(g() >> 11) * 0x1p-53), ks[s % 8]);
                if (x >= 1.0 - 0x1p-4 && x < 1.0 + 0x1.09p-4) continue;      // the routine's other branch
                xs.push_back(x);
                ref.push_back(log(x));
            }
            std::vector<Entry> next;
            for (const Entry &e : cand) {
                bool ok = true;
                for (size_t s = 0; s < xs.size() && ok; s++) ok = d2u(log_main(xs[s], e.invc, e.logc)) == d2u(ref[s]);
                if (ok) next.push_back(e);
            }
            cand.swap(next);
        }
        survivors[i] = (int)cand.size();
        if (!cand.empty()) table[i] = cand[0];
    }
    int bad = 0;
    for (int i = first; i < last; i++) {
        if (survivors[i] != 1) { fprintf(stderr, "subinterval %d: %d candidates survive\n", i, survivors[i]); bad++; }
        printf("0x%016llxull, 0x%016llxull,\n", (unsigned long long)d2u(table[i].invc), (unsigned long long)d2u(table[i].logc));
    }
    return bad != 0;
}
