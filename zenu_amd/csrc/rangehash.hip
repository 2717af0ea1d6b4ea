// rangehash.hip -- every f32 bit pattern of a range through a unary function of the library, folded
// into one 64-bit sum per block of patterns.  A host that folds its own libm's results the same way
// (one term per argument: argument and result bits through the finalizer of splitmix64, every NaN
// counted as one value) can compare every argument of the function with the device without copying
// a single result: equal sums, equal bits.  The functor is the one the elementwise kernels apply
// (elementwise.hpp), so what is checked is the arithmetic that ships.
#include "elementwise.hpp"

namespace zenu {
namespace {

__device__ __forceinline__ uint64_t range_hash_term(uint32_t arg_bits, uint32_t res_bits)
{
    if ((res_bits & 0x7fffffffu) > 0x7f800000u) res_bits = 0x7fc00000u;
    uint64_t z = ((uint64_t)arg_bits << 32) | res_bits;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

constexpr int kHashBlock = 256;

// the workgroup's terms added up (mod 2^64, so the order does not matter) and stored as the sum of its block
__device__ __forceinline__ void store_block_sum(uint64_t sum, uint64_t *sums)
{
    __shared__ uint64_t part[kHashBlock / 64];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = sum;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint64_t total = 0;
#pragma unroll
        for (int w = 0; w < kHashBlock / 64; w++) total += part[w];
        sums[blockIdx.x] = total;
    }
}

// one workgroup per block of 2^block_log2 f32 patterns, any functor over f32 (a unary function, powf with its exponent)
template <typename F>
__global__ __launch_bounds__(kHashBlock) void range_hash_functor_kernel(uint64_t first, int block_log2, uint64_t *sums, F f)
{
    f.init();
    const uint64_t per = 1ull << block_log2;
    const uint64_t start = first + (uint64_t)blockIdx.x * per;
    uint64_t sum = 0;
    for (uint64_t i = threadIdx.x; i < per; i += kHashBlock) {
        const uint32_t bits = (uint32_t)(start + i);
        const float x = __uint_as_float(bits);
        sum += range_hash_term(bits, __float_as_uint(f(x, x)));
    }
    store_block_sum(sum, sums);
}

template <int FN> int launch_range_hash(uint64_t first, uint64_t blocks, int block_log2, uint64_t *sums, hipStream_t s)
{
    range_hash_functor_kernel<UnaryF<float, FN>><<<(unsigned)blocks, kHashBlock, 0, s>>>(first, block_log2, sums,
                                                                                         UnaryF<float, FN>());
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

// f64: the arguments cannot be exhausted.  Argument number i has the high word i * step + offset (sign,
// exponent, 20 mantissa bits) and a pseudo-random low word that depends on i and `salt`; the term folds
// the argument's 64 bits, then the result's.
__device__ __forceinline__ uint64_t mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

__device__ __forceinline__ uint64_t range_arg_f64(uint64_t i, uint32_t step, uint32_t offset, uint64_t salt)
{
    const uint64_t hi = (uint32_t)(i * step + offset);
    const uint64_t lo = (uint32_t)(((i + salt) * 0x9E3779B97F4A7C15ull) >> 29);
    return (hi << 32) | lo;
}

template <typename F>
__global__ __launch_bounds__(kHashBlock) void range_hash_f64_kernel(uint64_t first, int block_log2, uint32_t step,
                                                                    uint32_t offset, uint64_t salt, uint64_t *sums, F f)
{
    f.init();
    const uint64_t per = 1ull << block_log2;
    const uint64_t start = first + (uint64_t)blockIdx.x * per;
    uint64_t sum = 0;
    for (uint64_t i = threadIdx.x; i < per; i += kHashBlock) {
        const uint64_t bits = range_arg_f64(start + i, step, offset, salt);
        const double x = __longlong_as_double((long long)bits);
        uint64_t rb = (uint64_t)__double_as_longlong(f(x, x));
        if ((rb & 0x7fffffffffffffffull) > 0x7ff0000000000000ull) rb = 0x7ff8000000000000ull;
        sum += mix64(mix64(bits) + rb);
    }
    store_block_sum(sum, sums);
}

template <int FN>
int launch_range_hash_f64(uint64_t first, uint64_t blocks, int block_log2, uint32_t step, uint32_t offset, uint64_t salt,
                          uint64_t *sums, hipStream_t s)
{
    range_hash_f64_kernel<UnaryF<double, FN>><<<(unsigned)blocks, kHashBlock, 0, s>>>(first, block_log2, step, offset, salt,
                                                                                      sums, UnaryF<double, FN>());
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

}  // namespace
}  // namespace zenu

using namespace zenu;

extern "C" int zenu_hip_unary_range_hash(int fn, uint64_t first, uint64_t count, int block_log2, uint64_t *sums_dev,
                                         zenu_stream_t stream)
{
    if (!sums_dev || block_log2 < 8 || block_log2 > 32) return ZENU_ERR_ARG;
    if ((count & ((1ull << block_log2) - 1)) || count == 0 || first + count > (1ull << 32)) return ZENU_ERR_ARG;
    const uint64_t blocks = count >> block_log2;
    if (blocks > 0x7fffffffull) return ZENU_ERR_UNSUPPORTED;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (fn) {
    case ZENU_EXP: return launch_range_hash<ZENU_EXP>(first, blocks, block_log2, sums_dev, s);
    case ZENU_LOG: return launch_range_hash<ZENU_LOG>(first, blocks, block_log2, sums_dev, s);
    case ZENU_TANH: return launch_range_hash<ZENU_TANH>(first, blocks, block_log2, sums_dev, s);
    case ZENU_SIGMOID: return launch_range_hash<ZENU_SIGMOID>(first, blocks, block_log2, sums_dev, s);
    case ZENU_SIN: return launch_range_hash<ZENU_SIN>(first, blocks, block_log2, sums_dev, s);
    case ZENU_COS: return launch_range_hash<ZENU_COS>(first, blocks, block_log2, sums_dev, s);
    case ZENU_TAN: return launch_range_hash<ZENU_TAN>(first, blocks, block_log2, sums_dev, s);
    case ZENU_ASIN: return launch_range_hash<ZENU_ASIN>(first, blocks, block_log2, sums_dev, s);
    case ZENU_ACOS: return launch_range_hash<ZENU_ACOS>(first, blocks, block_log2, sums_dev, s);
    case ZENU_ATAN: return launch_range_hash<ZENU_ATAN>(first, blocks, block_log2, sums_dev, s);
    case ZENU_SINH: return launch_range_hash<ZENU_SINH>(first, blocks, block_log2, sums_dev, s);
    case ZENU_COSH: return launch_range_hash<ZENU_COSH>(first, blocks, block_log2, sums_dev, s);
    default: return ZENU_ERR_ARG;
    }
}

extern "C" int zenu_hip_powf_range_hash(double exponent, uint64_t first, uint64_t count, int block_log2, uint64_t *sums_dev,
                                        zenu_stream_t stream)
{
    if (!sums_dev || block_log2 < 8 || block_log2 > 32) return ZENU_ERR_ARG;
    if ((count & ((1ull << block_log2) - 1)) || count == 0 || first + count > (1ull << 32)) return ZENU_ERR_ARG;
    const uint64_t blocks = count >> block_log2;
    if (blocks > 0x7fffffffull) return ZENU_ERR_UNSUPPORTED;
    PowF<float> f;
    f.s = (float)exponent;
    range_hash_functor_kernel<PowF<float>><<<(unsigned)blocks, kHashBlock, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        first, block_log2, sums_dev, f);
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

extern "C" int zenu_hip_unary_range_hash_f64(int fn, uint64_t first, uint64_t count, int block_log2, uint32_t step,
                                             uint32_t offset, uint64_t salt, uint64_t *sums_dev, zenu_stream_t stream)
{
    if (!sums_dev || block_log2 < 8 || block_log2 > 32 || step == 0) return ZENU_ERR_ARG;
    if ((count & ((1ull << block_log2) - 1)) || count == 0 || first + count > (1ull << 32)) return ZENU_ERR_ARG;
    const uint64_t blocks = count >> block_log2;
    if (blocks > 0x7fffffffull) return ZENU_ERR_UNSUPPORTED;
    hipStream_t s = reinterpret_cast<hipStream_t>(stream);
    switch (fn) {
    case ZENU_EXP: return launch_range_hash_f64<ZENU_EXP>(first, blocks, block_log2, step, offset, salt, sums_dev, s);
    case ZENU_TANH: return launch_range_hash_f64<ZENU_TANH>(first, blocks, block_log2, step, offset, salt, sums_dev, s);
    case ZENU_LOG: return launch_range_hash_f64<ZENU_LOG>(first, blocks, block_log2, step, offset, salt, sums_dev, s);
    case ZENU_SIN: return launch_range_hash_f64<ZENU_SIN>(first, blocks, block_log2, step, offset, salt, sums_dev, s);
    case ZENU_COS: return launch_range_hash_f64<ZENU_COS>(first, blocks, block_log2, step, offset, salt, sums_dev, s);
    case ZENU_SIGMOID: return launch_range_hash_f64<ZENU_SIGMOID>(first, blocks, block_log2, step, offset, salt, sums_dev, s);
    case ZENU_SINH: return launch_range_hash_f64<ZENU_SINH>(first, blocks, block_log2, step, offset, salt, sums_dev, s);
    case ZENU_COSH: return launch_range_hash_f64<ZENU_COSH>(first, blocks, block_log2, step, offset, salt, sums_dev, s);
    default: return ZENU_ERR_ARG;
    }
}


extern "C" int zenu_hip_powf_range_hash_f64(double exponent, uint64_t first, uint64_t count, int block_log2, uint32_t step,
                                            uint32_t offset, uint64_t salt, uint64_t *sums_dev, zenu_stream_t stream)
{
    if (!sums_dev || block_log2 < 8 || block_log2 > 32 || step == 0) return ZENU_ERR_ARG;
    if ((count & ((1ull << block_log2) - 1)) || count == 0 || first + count > (1ull << 32)) return ZENU_ERR_ARG;
    const uint64_t blocks = count >> block_log2;
    if (blocks > 0x7fffffffull) return ZENU_ERR_UNSUPPORTED;
    PowF<double> f;
    f.s = exponent;
    range_hash_f64_kernel<PowF<double>><<<(unsigned)blocks, kHashBlock, 0, reinterpret_cast<hipStream_t>(stream)>>>(
        first, block_log2, step, offset, salt, sums_dev, f);
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}
