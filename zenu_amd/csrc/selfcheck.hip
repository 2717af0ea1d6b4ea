// selfcheck.hip -- the short division and square root of zmath.hpp against the IEEE operations,
// on the device, on every f32 argument of every function that uses them.
//
// tanh, the sigmoid, sinh, cosh, tan, atan, asin and acos replace the compiler's 11-instruction IEEE
// division (and the square root) by a reciprocal estimate and one correction by the exact
// remainder.  That sequence is not correctly rounded for every operand pair, only for the pairs
// these functions feed it, and the only proof of that is exhaustive.  Here the header is
// instantiated twice -- as shipped, and with the IEEE operations in place of the short ones --
// and one launch per function walks all 2^32 bit patterns comparing the two results bit for bit:
// a few tens of milliseconds, so the check can run with every test run instead of waiting for an
// opt-in comparison with the host libm that takes the host minutes.  (That the IEEE build equals
// the host libm is what the host build of the header and the sampled device sweeps check.)
#include "common.hpp"
#include "zmath.hpp"

#define ZMATH_NAMESPACE zmath_ieee
#define ZMATH_EXACT_DIVISION
#include "zmath.hpp"
#undef ZMATH_EXACT_DIVISION
#undef ZMATH_NAMESPACE

namespace zenu {
namespace {

enum { kDivPairs = 1000, kSqrtArgs = 1001 };

#define ZENU_SELFCHECK_EVAL(NAME, NS)                                                                  \
    template <int FN> struct NAME {                                                                    \
        NS::ExpLog<float> m;                                                                           \
        NS::TanhRegs rg;                                                                               \
        NS::AtanfLds at;                                                                               \
        __device__ __forceinline__ void init()                                                         \
        {                                                                                              \
            if constexpr (FN == ZENU_SINH || FN == ZENU_COSH) m.init(true, false);                     \
            if constexpr (FN == ZENU_ATAN) at.init();                                                  \
            rg.pin();                                                                                  \
        }                                                                                              \
        __device__ __forceinline__ float operator()(uint32_t bits) const                               \
        {                                                                                              \
            const float x = __uint_as_float(bits);                                                     \
            if constexpr (FN == ZENU_TANH) return NS::tanhf_simd(x, rg);                               \
            else if constexpr (FN == ZENU_SIGMOID) return NS::sigmoidf_zenu(x, rg);                    \
            else if constexpr (FN == ZENU_SINH) return m.sinh(x, rg);                                  \
            else if constexpr (FN == ZENU_COSH) return m.cosh(x, rg);                                  \
            else if constexpr (FN == ZENU_ATAN) return NS::atanf_fdlibm(x, at.tab);                    \
            else if constexpr (FN == ZENU_ASIN) return NS::asinf_fdlibm(x);                            \
            else if constexpr (FN == ZENU_ACOS) return NS::acosf_fdlibm(x);                            \
            else if constexpr (FN == ZENU_TAN) return NS::tanf_glibc(x);                               \
            else if constexpr (FN == kDivPairs) {                                                      \
                /* arbitrary operands, every exponent: the short sequence has no operand scaling, */   \
                /* so quotients of very large or very small operands come out wrong               */   \
                const float a = __uint_as_float(bits * 2654435761u);                                   \
                const float b = __uint_as_float((bits ^ 0x9e3779b9u) * 2246822519u);                   \
                return NS::div_tanh(a, b);                                                             \
            } else {                                                                                   \
                return NS::sqrt_fast(__uint_as_float(bits & 0x7fffffffu));   /* subnormals included */ \
            }                                                                                          \
        }                                                                                              \
    };
ZENU_SELFCHECK_EVAL(EvalShort, zmath)
ZENU_SELFCHECK_EVAL(EvalIeee, zmath_ieee)

constexpr int kCheckBlock = 256;
constexpr unsigned kCheckGrid = 8192;

// every thread takes bit patterns tid, tid + nthreads, ...; result[0] += mismatches, result[1] = a bit pattern that differs
template <int FN>
__global__ __launch_bounds__(kCheckBlock) void selfcheck_kernel(unsigned long long *result)
{
    EvalShort<FN> f;
    EvalIeee<FN> g;
    f.init();
    g.init();
    const uint32_t nthreads = kCheckGrid * kCheckBlock;             // a power of two: 2^32 / nthreads patterns each
    const uint32_t tid = blockIdx.x * kCheckBlock + threadIdx.x;
    unsigned bad = 0;
    uint32_t first = 0;
    for (uint32_t k = 0; k < (uint32_t)(0x100000000ull / nthreads); k++) {
        const uint32_t bits = tid + k * nthreads;
        const uint32_t a = __float_as_uint(f(bits)), b = __float_as_uint(g(bits));
        if (a != b) {
            if (!bad) first = bits;
            bad++;
        }
    }
    if (bad) {
        atomicAdd(result, (unsigned long long)bad);
        atomicExch(result + 1, (unsigned long long)first | (1ull << 63));
    }
}

template <int FN> int run_check(unsigned long long *dev, hipStream_t s)
{
    selfcheck_kernel<FN><<<kCheckGrid, kCheckBlock, 0, s>>>(dev);
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

}  // namespace
}  // namespace zenu

using namespace zenu;

extern "C" int zenu_hip_selfcheck_short_division(int fn, uint64_t *mismatches, uint32_t *example_bits,
                                                 zenu_stream_t stream)
{
    if (!mismatches) return ZENU_ERR_ARG;
    int rc = ensure_init();
    if (rc) return rc;
    void *dev = nullptr;
    rc = zenu_hip_malloc(&dev, 16, stream);
    if (rc) return rc;
    rc = zenu_hip_memset_zero(dev, 16, stream);
    hipStream_t s = as_stream(stream);
    unsigned long long *d = static_cast<unsigned long long *>(dev);
    if (!rc) {
        switch (fn) {
        case ZENU_TANH: rc = run_check<ZENU_TANH>(d, s); break;
        case ZENU_SIGMOID: rc = run_check<ZENU_SIGMOID>(d, s); break;
        case ZENU_SINH: rc = run_check<ZENU_SINH>(d, s); break;
        case ZENU_COSH: rc = run_check<ZENU_COSH>(d, s); break;
        case ZENU_ATAN: rc = run_check<ZENU_ATAN>(d, s); break;
        case ZENU_ASIN: rc = run_check<ZENU_ASIN>(d, s); break;
        case ZENU_ACOS: rc = run_check<ZENU_ACOS>(d, s); break;
        case ZENU_TAN: rc = run_check<ZENU_TAN>(d, s); break;
        case kDivPairs: rc = run_check<kDivPairs>(d, s); break;
        case kSqrtArgs: rc = run_check<kSqrtArgs>(d, s); break;
        default: rc = ZENU_ERR_ARG;
        }
    }
    unsigned long long host[2] = {0, 0};
    if (!rc) rc = zenu_hip_memcpy_d2h(host, dev, 16, stream);     // blocking
    (void)zenu_hip_free(dev, stream);
    if (rc) return rc;
    *mismatches = host[0];
    if (example_bits) *example_bits = (uint32_t)host[1];
    return ZENU_OK;
}
