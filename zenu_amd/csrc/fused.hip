// fused.hip -- single-launch forms of the op chains ZeNu issues around a classifier head:
//   softmax_assign                  zenu-matrix/src/operation/softmax.rs:10-25
//                                   (x - max_axis(keep) ; exp ; sum(axis, keep) ; /= ; copy_from)
//   SoftMax::backward               zenu-autograd/src/loss/softmax.rs:33-40
//                                   (gx = y*gy ; sum(gx, axis, keep) ; gx - y*sum)
//   cross_entropy (+ its backward)  zenu-autograd/src/loss/cross_entropy.rs:12-23
//                                   (softmax(pred,1) ; log ; * ans ; sum_to([]) ; / -N)
//   Linear bias add + ReLU          zenu-layer/src/layers/linear.rs:27-31, zenu-autograd/src/activation/relu.rs:24-33
//
// Every element goes through the same sequence of individually rounded operations as in the
// chain (no contraction; f32 exp/log are the host libm's algorithm, zmath.hpp), so the fused results differ
// from the chain only where the chain itself is order dependent: the sums.  The "lines" kernels
// (one thread per softmax line) add in index order, exactly like sum.rs:20-25; the
// workgroup-per-row kernels add in a fixed tree.
//
// Geometry: operands are row-major [outer, R, inner] with the softmax axis R in the middle;
// views that are not in default stride are staged through a contiguous temporary.
#include <type_traits>
#include <math.h>

#include "common.hpp"
#include "vecmem.hpp"
#include "zmath.hpp"

namespace zenu {
namespace {

constexpr int kBlock = 256;
constexpr int kWaves = kBlock / 64;
constexpr int kLineMaxR = 64;   // rows up to this length: one thread per row
constexpr int kRegPacks = 4;    // workgroup-per-row: vectors a thread keeps in registers

// ---- workgroup reductions in a fixed order ------------------------------------------------------------

template <typename T, bool MAX> __device__ __forceinline__ T combine(T a, T b)
{
    if (MAX) return b > a ? b : a;   // a NaN never replaces (max.rs:27)
    return a + b;
}

template <typename T, bool MAX, int BLOCK = kBlock> __device__ __forceinline__ T block_red(T v, T *lds)
{
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = combine<T, MAX>(v, __shfl_xor(v, o));
    if (BLOCK == 64) return v;   // one wavefront: every lane already holds the result
    __syncthreads();   // lds may still be read from the previous reduction
    if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = v;
    __syncthreads();
    T r = lds[0];
#pragma unroll
    for (int w = 1; w < BLOCK / 64; w++) r = combine<T, MAX>(r, lds[w]);
    return r;
}

// ---- forward ---------------------------------------------------------------------------------------------
// CE: additionally rowloss[line] = sum_r target * log(softmax)   (inner == 1 only)

constexpr int kLineRegs = 16;   // lines up to this length are kept in registers by the lines kernel

template <typename T, bool CE>
__device__ __forceinline__ T softmax_line(const zmath::ExpLog<T> &ml, const T *x, T *y, int64_t line, int64_t R,
                                          int64_t inner, const T *target, T *rowloss);

// With `loss` set (cross-entropy, every line in this one workgroup) the kernel also folds the row
// terms and divides by -N, in the order of ce_finalize_kernel: the whole loss in one launch.
template <typename T, bool CE>
__global__ __launch_bounds__(kBlock) void softmax_lines_kernel(const T *x, T *y, int64_t lines, int64_t R,
                                                                int64_t inner, const T *target, T *rowloss,
                                                                T *loss, T neg_n)
{
    zmath::ExpLog<T> ml;
    ml.init(true, CE);
    const int64_t line = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    T row_term = (T)0;
    if (line < lines) row_term = softmax_line<T, CE>(ml, x, y, line, R, inner, target, rowloss);
    if constexpr (CE) {
        if (loss) {     // uniform: every thread of the workgroup gets here
            __shared__ T lds[kWaves];
            T acc = (T)0;
            if (line < lines) acc = acc + row_term;
            acc = block_red<T, false>(acc, lds);
            if (threadIdx.x == 0) *loss = acc / neg_n;
        }
    }
}

// one softmax line by one thread; returns the line's cross-entropy term (also stored to rowloss when set)
template <typename T, bool CE>
__device__ __forceinline__ T softmax_line(const zmath::ExpLog<T> &ml, const T *x, T *y, int64_t line, int64_t R,
                                          int64_t inner, const T *target, T *rowloss)
{
    int64_t q = line, c = 0;
    if (inner != 1) {
        q = line / inner;
        c = line - q * inner;
    }
    const int64_t base = q * R * inner + c;
    const T *xl = x + base;
    T *yl = y + base;
    if (R <= kLineRegs) {
        // a short line (the classes of a classifier head) stays in registers: its loads, and those of
        // the targets, are issued together instead of one per loop iteration, and nothing is read
        // back.  The operations and their order are those of the loops below.
        T v[kLineRegs], tg[kLineRegs];
#pragma unroll
        for (int r = 0; r < kLineRegs; r++) {
            const int64_t rl = r < R ? r : 0;
            v[r] = xl[rl * inner];
            if (CE) tg[r] = target[base + rl * inner];
        }
        T m = v[0];
#pragma unroll
        for (int r = 1; r < kLineRegs; r++)
            if (r < R && v[r] > m) m = v[r];
        T sum = (T)0;
#pragma unroll
        for (int r = 0; r < kLineRegs; r++) {
            if (r < R) {
                v[r] = ml.exp(v[r] - m);
                sum = sum + v[r];
            }
        }
        T acc = (T)0;
#pragma unroll
        for (int r = 0; r < kLineRegs; r++) {
            if (r < R) {
                const T s = v[r] / sum;
                yl[r * inner] = s;
                if (CE) acc = acc + tg[r] * ml.log(s);
            }
        }
        if (CE && rowloss) rowloss[line] = acc;
        return acc;
    }
    // max_axis: strict '>' from element 0 (max.rs:19-34)
    T m = xl[0];
    for (int64_t r = 1; r < R; r++) {
        const T v = xl[r * inner];
        if (v > m) m = v;
    }
    // exp(x - max), summed in index order starting from zero (sum.rs:20-25)
    T sum = (T)0;
    for (int64_t r = 0; r < R; r++) {
        const T e = ml.exp(xl[r * inner] - m);
        yl[r * inner] = e;
        sum = sum + e;
    }
    T acc = (T)0;
    for (int64_t r = 0; r < R; r++) {
        const T s = yl[r * inner] / sum;
        yl[r * inner] = s;
        if (CE) acc = acc + target[base + r * inner] * ml.log(s);
    }
    if (CE && rowloss) rowloss[line] = acc;
    return acc;
}

template <typename T, int VEC, bool CE, bool REG, bool NT, int kBlock = 256, int kRegPacks = 4>
__global__ __launch_bounds__(kBlock) void softmax_rows_kernel(const T *x, T *y, int64_t R, const T *target,
                                                               T *rowloss, zmath::ExpLog<T> ml)
{
    // (ml arrives as an argument so that the f64 constants of exp / log sit in scalar registers; written
    // as literals each is copied into a register pair per use, and this kernel is bound by its scalar
    // instructions: the branch-free exp for the same reason)
    __shared__ T lds[4];
    if (!REG) ml.init(true, CE);
    const int64_t row = blockIdx.x;
    const T *xr = x + row * R;
    T *yr = y + row * R;
    const T *tr = CE ? target + row * R : nullptr;
    const int64_t first = (int64_t)threadIdx.x * VEC;
    constexpr int64_t step = (int64_t)kBlock * VEC;
    const T x0 = xr[0];
    T acc = (T)0;

    if (REG) {   // R <= kRegPacks * step: the row lives in registers, one read and one write
        Pack<T, VEC> v[kRegPacks];
        T m = -INFINITY;
#pragma unroll
        for (int k = 0; k < kRegPacks; k++) {
            const int64_t r = first + k * step;
            v[k] = r < R ? load_pack<T, VEC, NT>(xr + r) : splat<T, VEC>(-INFINITY);
#pragma unroll
            for (int j = 0; j < VEC; j++) m = combine<T, true>(m, v[k].v[j]);
        }
        // the targets of the cross-entropy terms travel with the row: loaded where they are used, each
        // pack cost the end of the kernel a round trip of its own
        Pack<T, VEC> tg[kRegPacks];
        if (CE) {
#pragma unroll
            for (int k = 0; k < kRegPacks; k++) {
                const int64_t r = first + k * step;
                tg[k] = load_pack<T, VEC, NT>(tr + (r < R ? r : 0));
            }
        }
        ml.init(true, CE);      // after the row's loads are issued: the table fetch overlaps them
        m = block_red<T, true, kBlock>(m, lds);
        if (x0 != x0) m = x0;   // a NaN in position 0 is never replaced
        T sum = (T)0;
        T least = INFINITY;     // the smallest of this thread's terms
#pragma unroll
        for (int k = 0; k < kRegPacks; k++) {
            if (first + k * step < R) {
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    v[k].v[j] = ml.exp_flat(v[k].v[j] - m);
                    sum = sum + v[k].v[j];
                    least = v[k].v[j] < least ? v[k].v[j] : least;
                }
            }
        }
        sum = block_red<T, false, kBlock>(sum, lds);
        // Every quotient of the row has the same divisor.  With r = RN(1 / sum): q0 = RN(a r), the
        // exact remainder a - sum q0 (one fma) and q = fma(remainder, r, q0) is the correctly rounded
        // a / sum (Markstein) unless the divisor's mantissa is all ones, as long as nothing underflows:
        // three instructions per element instead of the division's eleven.  The thread takes that road
        // when its terms are at least 2^-64 and the sum lies in [1, 2^23) (quotient and remainder stay
        // normal); otherwise it divides.  On 9.6e9 random pairs from those ranges (terms down to 2^-80)
        // the host finds no quotient that differs from the division's.
        bool shared_divisor = false;
        if constexpr (sizeof(T) == 4) {
            uint32_t sb;
            __builtin_memcpy(&sb, &sum, 4);
            shared_divisor = least >= (T)0x1p-64f && sum >= (T)1 && sum < (T)0x1p23f && (sb & 0x7fffffu) != 0x7fffffu;
        }
        auto finish = [&](auto by_reciprocal) {
            const T rcp = decltype(by_reciprocal)::value ? (T)1 / sum : (T)0;
#pragma unroll
            for (int k = 0; k < kRegPacks; k++) {
                const int64_t r = first + k * step;
                if (r < R) {
                    const Pack<T, VEC> t = tg[k];
#pragma unroll
                    for (int j = 0; j < VEC; j++) {
                        T s;
                        if constexpr (decltype(by_reciprocal)::value && sizeof(T) == 4) {
                            const float a = v[k].v[j];
                            const float q0 = a * rcp;
                            s = __builtin_fmaf(__builtin_fmaf(-sum, q0, a), rcp, q0);
                        } else {
                            s = v[k].v[j] / sum;
                        }
                        v[k].v[j] = s;
                        if (CE) acc = acc + t.v[j] * ml.log(s);
                    }
                    // the CE output is read again by the backward pass; plain softmax is one stream in, one out
                    if constexpr (NT && !CE && VEC > 1) store_pack_wt<T, VEC>(yr + r, v[k]);
                    else store_pack<T, VEC, false>(yr + r, v[k]);
                }
            }
        };
        if (shared_divisor) finish(std::true_type());
        else finish(std::false_type());
    } else {     // long rows: three passes; the second and third find the row in cache
        T m = -INFINITY;
        for (int64_t r = first; r < R; r += step) {
            const Pack<T, VEC> v = load_pack<T, VEC, false>(xr + r);
#pragma unroll
            for (int j = 0; j < VEC; j++) m = combine<T, true>(m, v.v[j]);
        }
        m = block_red<T, true, kBlock>(m, lds);
        if (x0 != x0) m = x0;
        T sum = (T)0;
        for (int64_t r = first; r < R; r += step) {
            Pack<T, VEC> v = load_pack<T, VEC, false>(xr + r);
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                v.v[j] = ml.exp_flat(v.v[j] - m);
                sum = sum + v.v[j];
            }
            store_pack<T, VEC, false>(yr + r, v);
        }
        sum = block_red<T, false, kBlock>(sum, lds);
        for (int64_t r = first; r < R; r += step) {   // each thread re-reads what it wrote itself
            Pack<T, VEC> v = load_pack<T, VEC, false>(yr + r);
            Pack<T, VEC> t;
            if (CE) t = load_pack<T, VEC, false>(tr + r);
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                const T s = v.v[j] / sum;
                v.v[j] = s;
                if (CE) acc = acc + t.v[j] * ml.log(s);
            }
            store_pack<T, VEC, false>(yr + r, v);
        }
    }
    if (CE) {
        acc = block_red<T, false, kBlock>(acc, lds);
        if (threadIdx.x == 0) rowloss[row] = acc;
    }
}

// loss = (sum of the row terms) / (-N), one workgroup
template <typename T>
__global__ __launch_bounds__(kBlock) void ce_finalize_kernel(const T *rowloss, int64_t n, T *loss, T neg_n)
{
    __shared__ T lds[kWaves];
    T acc = (T)0;
    int64_t i = threadIdx.x;
    for (; i + 7 * kBlock < n; i += 8 * kBlock) {       // eight loads in flight, added in index order
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; u++) v[u] = rowloss[i + u * kBlock];
#pragma unroll
        for (int u = 0; u < 8; u++) acc = acc + v[u];
    }
    for (; i < n; i += kBlock) acc = acc + rowloss[i];
    acc = block_red<T, false>(acc, lds);
    if (threadIdx.x == 0) *loss = acc / neg_n;
}

// ---- backward --------------------------------------------------------------------------------------------
// gx = t - y * sum(t), t = y * gy.  CE: gy = (target * g_total) / y with g_total = gout / (-N), the
// chain div -> sum_to -> mul -> log backward of cross_entropy.rs:18-22.

template <typename T, bool CE> struct GySource {
    const T *p;        // gy, or the target when CE
    T g_total;
    __device__ __forceinline__ T get(int64_t off, T yv) const
    {
        if (CE) return (p[off] * g_total) / yv;
        return p[off];
    }
};

// With `colsum` set (every line in this one workgroup, lines of at most kLineRegs elements, inner == 1)
// the kernel also writes the column sums of gx -- the bias gradient of the Linear layer that
// produced the logits (zenu-layer/src/layers/linear.rs:27-31 through the `sum_to` of
// zenu-autograd/src/lib.rs:466-486) -- each folded over the lines in the fixed order of block_red.
template <typename T, bool CE>
__global__ __launch_bounds__(kBlock) void softmax_bwd_lines_kernel(const T *y, const T *gy_or_target, T *gx,
                                                                    int64_t lines, int64_t R, int64_t inner,
                                                                    const T *gout, T neg_n, T *colsum)
{
    const int64_t line = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (colsum) {    // uniform; the host sends this only with R <= kLineRegs, inner == 1, one workgroup
        __shared__ T lds[kLineRegs * kWaves];
        const bool active = line < lines;
        const T g_total = CE ? (gout ? *gout : (T)1) / neg_n : (T)0;
        const int64_t base = (active ? line : 0) * R;
        T yv[kLineRegs], pv[kLineRegs], t[kLineRegs];
#pragma unroll
        for (int r = 0; r < kLineRegs; r++) {
            const int64_t off = base + (r < R ? r : 0);
            yv[r] = y[off];
            pv[r] = gy_or_target[off];
        }
        T sum = (T)0;
#pragma unroll
        for (int r = 0; r < kLineRegs; r++) {
            if (r < R) {
                t[r] = yv[r] * (CE ? (pv[r] * g_total) / yv[r] : pv[r]);
                sum = sum + t[r];
            }
        }
        // the column sums in the order of block_red (butterfly inside a wavefront, then the wavefronts
        // in index order), all columns behind ONE barrier instead of two per column
#pragma unroll
        for (int r = 0; r < kLineRegs; r++) {
            if (r < R) {
                const T g = t[r] - yv[r] * sum;
                if (active) gx[base + r] = g;
                T c = (T)0;
                if (active) c = c + g;
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) c = c + __shfl_xor(c, o);
                if ((threadIdx.x & 63) == 0) lds[r * kWaves + (threadIdx.x >> 6)] = c;
            }
        }
        __syncthreads();
        if ((int64_t)threadIdx.x < R) {
            T c = lds[threadIdx.x * kWaves];
#pragma unroll
            for (int w = 1; w < kWaves; w++) c = c + lds[threadIdx.x * kWaves + w];
            colsum[threadIdx.x] = c;
        }
        return;
    }
    if (line >= lines) return;
    GySource<T, CE> src;
    src.p = gy_or_target;
    src.g_total = CE ? (gout ? *gout : (T)1) / neg_n : (T)0;
    int64_t q = line, c = 0;
    if (inner != 1) {
        q = line / inner;
        c = line - q * inner;
    }
    const int64_t base = q * R * inner + c;
    if (R <= kLineRegs) {     // a short line in registers, as in the forward kernel: same operations, same order
        T yv[kLineRegs], pv[kLineRegs], t[kLineRegs];
#pragma unroll
        for (int r = 0; r < kLineRegs; r++) {
            const int64_t off = base + (r < R ? r : 0) * inner;
            yv[r] = y[off];
            pv[r] = gy_or_target[off];
        }
        T sum = (T)0;
#pragma unroll
        for (int r = 0; r < kLineRegs; r++) {
            if (r < R) {
                t[r] = yv[r] * (CE ? (pv[r] * src.g_total) / yv[r] : pv[r]);
                sum = sum + t[r];
            }
        }
#pragma unroll
        for (int r = 0; r < kLineRegs; r++)
            if (r < R) gx[base + r * inner] = t[r] - yv[r] * sum;
        return;
    }
    T sum = (T)0;
    for (int64_t r = 0; r < R; r++) {
        const int64_t off = base + r * inner;
        const T yv = y[off];
        const T t = yv * src.get(off, yv);
        gx[off] = t;
        sum = sum + t;
    }
    for (int64_t r = 0; r < R; r++) {
        const int64_t off = base + r * inner;
        gx[off] = gx[off] - y[off] * sum;
    }
}

template <typename T, int VEC, bool CE, bool REG, bool NT>
__global__ __launch_bounds__(kBlock) void softmax_bwd_rows_kernel(const T *y, const T *gy_or_target, T *gx,
                                                                   int64_t R, const T *gout, T neg_n)
{
    __shared__ T lds[kWaves];
    const T g_total = CE ? (gout ? *gout : (T)1) / neg_n : (T)0;
    const int64_t base = (int64_t)blockIdx.x * R;
    const T *yr = y + base;
    const T *sr = gy_or_target + base;
    T *gr = gx + base;
    const int64_t first = (int64_t)threadIdx.x * VEC;
    constexpr int64_t step = (int64_t)kBlock * VEC;
    T sum = (T)0;
    if (REG) {   // the row of y and of t = y * gy stays in registers: two reads, one write
        Pack<T, VEC> yv[kRegPacks], gv[kRegPacks], t[kRegPacks];
        // all loads of the thread first (a pack past the end of the row reads the row's first one and
        // is not used): with the loads inside the bounds check the compiler waits for each pair
        // before it issues the next, because the running sum orders the blocks
#pragma unroll
        for (int k = 0; k < kRegPacks; k++) {
            const int64_t r = first + k * step;
            const int64_t rl = r < R ? r : 0;
            yv[k] = load_pack<T, VEC, NT && !CE>(yr + rl);
            gv[k] = load_pack<T, VEC, NT>(sr + rl);
        }
#pragma unroll
        for (int k = 0; k < kRegPacks; k++) {
            const int64_t r = first + k * step;
            if (r < R) {
                const Pack<T, VEC> g = gv[k];
#pragma unroll
                for (int j = 0; j < VEC; j++) {
                    const T gyv = CE ? (g.v[j] * g_total) / yv[k].v[j] : g.v[j];
                    t[k].v[j] = yv[k].v[j] * gyv;
                    sum = sum + t[k].v[j];
                }
            }
        }
        sum = block_red<T, false>(sum, lds);
#pragma unroll
        for (int k = 0; k < kRegPacks; k++) {
            const int64_t r = first + k * step;
            if (r < R) {
#pragma unroll
                for (int j = 0; j < VEC; j++) t[k].v[j] = t[k].v[j] - yv[k].v[j] * sum;
                store_pack<T, VEC, NT>(gr + r, t[k]);
            }
        }
    } else {     // long rows: t goes to gx first; the second pass finds both rows in cache
        for (int64_t r = first; r < R; r += step) {
            const Pack<T, VEC> yv = load_pack<T, VEC, false>(yr + r);
            const Pack<T, VEC> g = load_pack<T, VEC, false>(sr + r);
            Pack<T, VEC> t;
#pragma unroll
            for (int j = 0; j < VEC; j++) {
                const T gyv = CE ? (g.v[j] * g_total) / yv.v[j] : g.v[j];
                t.v[j] = yv.v[j] * gyv;
                sum = sum + t.v[j];
            }
            store_pack<T, VEC, false>(gr + r, t);
        }
        sum = block_red<T, false>(sum, lds);
        for (int64_t r = first; r < R; r += step) {
            const Pack<T, VEC> yv = load_pack<T, VEC, false>(yr + r);
            Pack<T, VEC> t = load_pack<T, VEC, false>(gr + r);
#pragma unroll
            for (int j = 0; j < VEC; j++) t.v[j] = t.v[j] - yv.v[j] * sum;
            store_pack<T, VEC, false>(gr + r, t);
        }
    }
}

// ---- a classifier head's batch in ONE workgroup, four lanes per line -------------------------------------------
// lines <= 256 of R <= 16 elements, contiguous (inner == 1).  One thread per line (the lines kernels
// above) is a single wavefront per SIMD walking through 16 unrolled copies of exp / log / division:
// 7-8 us for [256,10], most of it instruction fetch and dependent latencies that nothing overlaps.
// Here a quad of lanes owns a line -- lane q holds elements q, q + 4, q + 8, q + 12 -- in a workgroup
// of 1024 threads: four copies of the transcendental code, sixteen wavefronts.  Everything that the
// one-thread form does in index order (the max scan, the sum of the exponentials, the sum of the
// cross-entropy terms, the sum of t) is still done in index order, by every lane of the quad on
// values gathered from its neighbours, so the bits are the same.
constexpr int kHeadBlock = 1024;
constexpr int kHeadLines = kHeadBlock / 4;
constexpr int kHeadOwn = kLineRegs / 4;

// full[r] for r = 4 i + q is own[i] of lane q of the quad
template <typename T> __device__ __forceinline__ void quad_gather(const T (&own)[kHeadOwn], T (&full)[kLineRegs])
{
#pragma unroll
    for (int i = 0; i < kHeadOwn; i++) {
#pragma unroll
        for (int q = 0; q < 4; q++) full[4 * i + q] = __shfl(own[i], q, 4);
    }
}

// Forward: y = softmax(x) per line, *loss = sum over lines of (sum_r target * log y) / neg_n, the row
// terms folded as ce_finalize_kernel folds them (256 lanes: butterfly per wavefront, wavefronts in order).
template <typename T>
__global__ __launch_bounds__(kHeadBlock) void ce_head_forward_kernel(const T *x, T *y, int64_t lines, int64_t R,
                                                                      const T *target, T *loss, T neg_n)
{
    __shared__ T terms[kHeadLines];
    __shared__ T wave_sum[kHeadLines / 64];
    const int q = threadIdx.x & 3;
    const int64_t line = threadIdx.x >> 2;
    const bool active = line < lines;
    const int64_t base = (active ? line : 0) * R;
    T v[kHeadOwn], tg[kHeadOwn];
#pragma unroll
    for (int i = 0; i < kHeadOwn; i++) {
        const int r = 4 * i + q;
        const int64_t off = base + (r < R ? r : 0);
        v[i] = x[off];
        tg[i] = target[off];
    }
    zmath::ExpLog<T> ml;
    ml.init(true, true);
    T full[kLineRegs];
    quad_gather<T>(v, full);
    T m = full[0];                       // max_axis: strict '>' from element 0 (max.rs:19-34)
#pragma unroll
    for (int r = 1; r < kLineRegs; r++)
        if (r < R && full[r] > m) m = full[r];
#pragma unroll
    for (int i = 0; i < kHeadOwn; i++) v[i] = ml.exp(v[i] - m);
    quad_gather<T>(v, full);
    T sum = (T)0;                        // in index order from zero (sum.rs:20-25)
#pragma unroll
    for (int r = 0; r < kLineRegs; r++)
        if (r < R) sum = sum + full[r];
    T term[kHeadOwn];
#pragma unroll
    for (int i = 0; i < kHeadOwn; i++) {
        const int r = 4 * i + q;
        const T sm = v[i] / sum;
        if (active && r < R) y[base + r] = sm;
        term[i] = r < R ? tg[i] * ml.log(sm) : (T)0;
    }
    quad_gather<T>(term, full);
    T acc = (T)0;
#pragma unroll
    for (int r = 0; r < kLineRegs; r++)
        if (r < R) acc = acc + full[r];
    if (q == 0) terms[line] = active ? (T)0 + acc : (T)0;
    __syncthreads();
    if (threadIdx.x < kHeadLines) {      // uniform per wavefront
        T a = terms[threadIdx.x];
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) a = a + __shfl_xor(a, o);
        if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = a;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        T a = wave_sum[0];
#pragma unroll
        for (int w = 1; w < kHeadLines / 64; w++) a = a + wave_sum[w];
        *loss = a / neg_n;
    }
}

// Backward: gx = t - y * sum(t) with t = y * ((target * g_total) / y), and colsum[r] = the sum of gx over
// the lines (when set), each column folded as block_red folds 256 lanes.
template <typename T>
__global__ __launch_bounds__(kHeadBlock) void ce_head_backward_kernel(const T *y, const T *target, T *gx, int64_t lines,
                                                                       int64_t R, const T *gout, T neg_n, T *colsum)
{
    __shared__ T cols[kLineRegs][kHeadLines];      // gx by column, for the column sums
    const int q = threadIdx.x & 3;
    const int64_t line = threadIdx.x >> 2;
    const bool active = line < lines;
    const int64_t base = (active ? line : 0) * R;
    const T g_total = (gout ? *gout : (T)1) / neg_n;
    T yv[kHeadOwn], t[kHeadOwn];
#pragma unroll
    for (int i = 0; i < kHeadOwn; i++) {
        const int r = 4 * i + q;
        const int64_t off = base + (r < R ? r : 0);
        yv[i] = y[off];
        t[i] = target[off];
    }
#pragma unroll
    for (int i = 0; i < kHeadOwn; i++) t[i] = yv[i] * ((t[i] * g_total) / yv[i]);
    T full[kLineRegs];
    quad_gather<T>(t, full);
    T sum = (T)0;
#pragma unroll
    for (int r = 0; r < kLineRegs; r++)
        if (r < R) sum = sum + full[r];
#pragma unroll
    for (int i = 0; i < kHeadOwn; i++) {
        const int r = 4 * i + q;
        const T g = t[i] - yv[i] * sum;
        if (active && r < R) gx[base + r] = g;
        if (colsum && r < R) cols[r][line] = active ? (T)0 + g : (T)0;
    }
    if (!colsum) return;                 // uniform
    __syncthreads();
    // wavefront w folds column w: four runs of 64 lines, each with the butterfly, then the runs in order
    const int64_t col = threadIdx.x >> 6;
    if (col < R) {
        const int lane = threadIdx.x & 63;
        T total = (T)0;
#pragma unroll
        for (int w = 0; w < kHeadLines / 64; w++) {
            T c = cols[col][w * 64 + lane];
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) c = c + __shfl_xor(c, o);
            total = w == 0 ? c : total + c;
        }
        if (lane == 0) colsum[col] = total;
    }
}

// ---- bias add + ReLU ----------------------------------------------------------------------------------------
// pre = z + bias (broadcast over rows), act = pre > 0 ? pre : alpha * pre  (relu.rs:44-48)

template <typename T, int VEC>
__global__ __launch_bounds__(kBlock) void bias_relu_kernel(const T *z, const T *bias, T *pre, T *act,
                                                            int64_t rows, int64_t packs_per_row, T alpha)
{
    const int64_t total = rows * packs_per_row;
    for (int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (int64_t)gridDim.x * kBlock) {
        const int64_t row = i / packs_per_row;
        const int64_t col = (i - row * packs_per_row) * VEC;
        const int64_t off = i * VEC;
        const Pack<T, VEC> v = load_pack<T, VEC, false>(z + off);
        const Pack<T, VEC> b = load_pack<T, VEC, false>(bias + col);
        Pack<T, VEC> a, h;
#pragma unroll
        for (int j = 0; j < VEC; j++) {
            a.v[j] = v.v[j] + b.v[j];
            h.v[j] = a.v[j] > (T)0 ? a.v[j] : alpha * a.v[j];
        }
        if (pre) store_pack<T, VEC, false>(pre + off, a);
        store_pack<T, VEC, false>(act + off, h);
    }
}

// Rows that are a whole number of 64-lane vectors: a 64-thread workgroup per contiguous piece of a
// row, one vector per lane (the shape that streams best when most of the traffic is stores); the
// row / column split is one 32-bit division per workgroup on the scalar unit.
constexpr int kTileLanes = 64;
template <typename T, int VEC, bool NT>
__global__ __launch_bounds__(kTileLanes) void bias_relu_tile_kernel(const T *z, const T *bias, T *pre, T *act,
                                                                     uint32_t tiles_per_row, T alpha)
{
    const uint32_t row = blockIdx.x / tiles_per_row;
    const uint32_t tile = blockIdx.x - row * tiles_per_row;
    const int64_t col = ((int64_t)tile * kTileLanes + threadIdx.x) * VEC;
    const int64_t off = (int64_t)blockIdx.x * kTileLanes * VEC + (int64_t)threadIdx.x * VEC;
    const Pack<T, VEC> v = load_pack<T, VEC, NT>(z + off);
    const Pack<T, VEC> b = load_pack<T, VEC, false>(bias + col);
    Pack<T, VEC> a, h;
#pragma unroll
    for (int j = 0; j < VEC; j++) {
        a.v[j] = v.v[j] + b.v[j];
        h.v[j] = a.v[j] > (T)0 ? a.v[j] : alpha * a.v[j];
    }
    if constexpr (NT && VEC > 1) {
        if (pre) store_pack_wt<T, VEC>(pre + off, a);
        store_pack_wt<T, VEC>(act + off, h);
    } else {
        if (pre) store_pack<T, VEC, NT>(pre + off, a);
        store_pack<T, VEC, NT>(act + off, h);
    }
}

// ---- host side ------------------------------------------------------------------------------------------------

// a tensor as a contiguous device buffer: itself, or a temporary copy
template <typename T> struct ContigIn {
    Workspace ws;
    const T *ptr;
    int status;
    ContigIn(const zenu_tensor_t &t, int dtype, hipStream_t s)
        : ws(is_default_stride_strict(t) ? 0 : (size_t)num_elm(t) * sizeof(T), s),
          ptr(static_cast<const T *>(t.ptr)), status(ws.status)
    {
        if (is_default_stride_strict(t) || status) return;
        zenu_tensor_t tmp = default_view(ws.ptr, t.ndim, t.shape);
        status = zenu_hip_copy(dtype, &tmp, &t, reinterpret_cast<zenu_stream_t>(s));
        ptr = static_cast<const T *>(ws.ptr);
    }
};

// a contiguous buffer to write into: the tensor itself, or a temporary that finish() copies out
template <typename T> struct ContigOut {
    Workspace ws;
    const zenu_tensor_t &t;
    T *ptr;
    int status;
    int dtype;
    bool temp;
    ContigOut(const zenu_tensor_t &t_, int dtype_, hipStream_t s)
        : ws(is_default_stride_strict(t_) ? 0 : (size_t)num_elm(t_) * sizeof(T), s), t(t_),
          ptr(static_cast<T *>(t_.ptr)), status(ws.status), dtype(dtype_), temp(!is_default_stride_strict(t_))
    {
        if (temp && !status) ptr = static_cast<T *>(ws.ptr);
    }
    int finish()
    {
        if (!temp) return ZENU_OK;
        zenu_tensor_t tmp = default_view(ws.ptr, t.ndim, t.shape);
        return zenu_hip_copy(dtype, &t, &tmp, reinterpret_cast<zenu_stream_t>(ws.stream));
    }
};

struct Geometry { int64_t outer, R, inner; };

Geometry geometry(const zenu_tensor_t &t, int axis)
{
    Geometry g = {1, t.shape[axis], 1};
    for (int i = 0; i < axis; i++) g.outer *= t.shape[i];
    for (int i = axis + 1; i < t.ndim; i++) g.inner *= t.shape[i];
    return g;
}

inline bool grid_ok(int64_t blocks) { return blocks > 0 && blocks <= 0x7fffffffLL; }

// true when the cross-entropy forward of this geometry is one workgroup of the lines kernel, which
// then also produces the loss (no row terms in memory, no second launch)
inline bool ce_single_workgroup(const Geometry &g)
{
    return g.inner == 1 && g.R <= kLineMaxR && g.outer <= kBlock;
}

template <typename T, bool CE>
int softmax_forward_launch(const T *x, T *y, Geometry g, const T *target, T *rowloss, hipStream_t s,
                           T *loss = nullptr, T neg_n = (T)0)
{
    constexpr int VEC = VecOf<T>::N;
    const int64_t lines = g.outer * g.inner;
    if constexpr (CE) {
        if (loss && g.inner == 1 && g.R <= kLineRegs && lines <= kHeadLines) {   // a classifier head: four lanes per line
            ce_head_forward_kernel<T><<<1, kHeadBlock, 0, s>>>(x, y, lines, g.R, target, loss, neg_n);
            ZENU_LAUNCH_CHECK();
            return ZENU_OK;
        }
    }
    if (g.inner != 1 || g.R <= kLineMaxR) {
        const int64_t blocks = (lines + kBlock - 1) / kBlock;
        if (!grid_ok(blocks)) return ZENU_ERR_UNSUPPORTED;
        T *fold = (CE && blocks == 1) ? loss : nullptr;
        softmax_lines_kernel<T, CE><<<(unsigned)blocks, kBlock, 0, s>>>(x, y, lines, g.R, g.inner, target, rowloss, fold, neg_n);
    } else {
        if (!grid_ok(lines)) return ZENU_ERR_UNSUPPORTED;
        const bool vec = g.R % VEC == 0 && aligned16(x) && aligned16(y) && (!CE || aligned16(target));
        const bool reg = g.R <= (int64_t)kRegPacks * kBlock * (vec ? VEC : 1);
        const unsigned grid = (unsigned)lines;
        const bool nt = vec && reg && lines * g.R * (int64_t)sizeof(T) * 2 >= kStreamBytes;
        // (one wavefront or 128 threads per row with more vectors per lane measured 4-9 % slower)
        if (nt)               softmax_rows_kernel<T, VEC, CE, true, true><<<grid, kBlock, 0, s>>>(x, y, g.R, target, rowloss, zmath::ExpLog<T>());
        else if (vec && reg)  softmax_rows_kernel<T, VEC, CE, true, false><<<grid, kBlock, 0, s>>>(x, y, g.R, target, rowloss, zmath::ExpLog<T>());
        else if (vec)         softmax_rows_kernel<T, VEC, CE, false, false><<<grid, kBlock, 0, s>>>(x, y, g.R, target, rowloss, zmath::ExpLog<T>());
        else if (reg)         softmax_rows_kernel<T, 1, CE, true, false><<<grid, kBlock, 0, s>>>(x, y, g.R, target, rowloss, zmath::ExpLog<T>());
        else                  softmax_rows_kernel<T, 1, CE, false, false><<<grid, kBlock, 0, s>>>(x, y, g.R, target, rowloss, zmath::ExpLog<T>());
    }
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

template <typename T, bool CE>
int softmax_backward_launch(const T *y, const T *gy_or_target, T *gx, Geometry g, const T *gout, T neg_n,
                            hipStream_t s, T *colsum = nullptr)
{
    const int64_t lines = g.outer * g.inner;
    if (colsum && !(g.inner == 1 && g.R <= kLineRegs && lines <= kBlock)) return ZENU_ERR_UNSUPPORTED;
    if constexpr (CE) {
        if (g.inner == 1 && g.R <= kLineRegs && lines <= kHeadLines) {           // a classifier head: four lanes per line
            ce_head_backward_kernel<T><<<1, kHeadBlock, 0, s>>>(y, gy_or_target, gx, lines, g.R, gout, neg_n, colsum);
            ZENU_LAUNCH_CHECK();
            return ZENU_OK;
        }
    }
    if (g.inner != 1 || g.R <= kLineMaxR) {
        const int64_t blocks = (lines + kBlock - 1) / kBlock;
        if (!grid_ok(blocks)) return ZENU_ERR_UNSUPPORTED;
        softmax_bwd_lines_kernel<T, CE><<<(unsigned)blocks, kBlock, 0, s>>>(y, gy_or_target, gx, lines, g.R, g.inner,
                                                                             gout, neg_n, colsum);
    } else {
        if (!grid_ok(lines)) return ZENU_ERR_UNSUPPORTED;
        constexpr int VEC = VecOf<T>::N;
        const bool vec = g.R % VEC == 0 && aligned16(y) && aligned16(gy_or_target) && aligned16(gx);
        const bool reg = g.R <= (int64_t)kRegPacks * kBlock * (vec ? VEC : 1);
        const bool nt = vec && reg && lines * g.R * (int64_t)sizeof(T) * 3 >= kStreamBytes;
        const unsigned grid = (unsigned)lines;
        if (nt)              softmax_bwd_rows_kernel<T, VEC, CE, true, true><<<grid, kBlock, 0, s>>>(y, gy_or_target, gx, g.R, gout, neg_n);
        else if (vec && reg) softmax_bwd_rows_kernel<T, VEC, CE, true, false><<<grid, kBlock, 0, s>>>(y, gy_or_target, gx, g.R, gout, neg_n);
        else if (vec)        softmax_bwd_rows_kernel<T, VEC, CE, false, false><<<grid, kBlock, 0, s>>>(y, gy_or_target, gx, g.R, gout, neg_n);
        else if (reg)        softmax_bwd_rows_kernel<T, 1, CE, true, false><<<grid, kBlock, 0, s>>>(y, gy_or_target, gx, g.R, gout, neg_n);
        else                 softmax_bwd_rows_kernel<T, 1, CE, false, false><<<grid, kBlock, 0, s>>>(y, gy_or_target, gx, g.R, gout, neg_n);
    }
    ZENU_LAUNCH_CHECK();
    return ZENU_OK;
}

template <typename T>
int softmax_t(int dtype, const zenu_tensor_t &to, const zenu_tensor_t &src, int axis, hipStream_t s)
{
    if (num_elm(src) == 0) return ZENU_OK;
    ContigIn<T> in(src, dtype, s);
    if (in.status) return in.status;
    ContigOut<T> out(to, dtype, s);
    if (out.status) return out.status;
    int rc = softmax_forward_launch<T, false>(in.ptr, out.ptr, geometry(src, axis), nullptr, nullptr, s);
    return rc ? rc : out.finish();
}

template <typename T>
int softmax_backward_t(int dtype, const zenu_tensor_t &gx, const zenu_tensor_t &y, const zenu_tensor_t &gy,
                       int axis, hipStream_t s)
{
    if (num_elm(y) == 0) return ZENU_OK;
    ContigIn<T> yin(y, dtype, s);
    if (yin.status) return yin.status;
    ContigIn<T> gin(gy, dtype, s);
    if (gin.status) return gin.status;
    ContigOut<T> out(gx, dtype, s);
    if (out.status) return out.status;
    int rc = softmax_backward_launch<T, false>(yin.ptr, gin.ptr, out.ptr, geometry(y, axis), nullptr, (T)0, s);
    return rc ? rc : out.finish();
}

template <typename T>
int cross_entropy_t(int dtype, const zenu_tensor_t &loss, const zenu_tensor_t &prob, const zenu_tensor_t &pred,
                    const zenu_tensor_t &ans, hipStream_t s)
{
    const int64_t n = pred.shape[0];
    if (num_elm(pred) == 0) return ZENU_ERR_SHAPE;
    ContigIn<T> in(pred, dtype, s);
    if (in.status) return in.status;
    ContigIn<T> tin(ans, dtype, s);
    if (tin.status) return tin.status;
    ContigOut<T> out(prob, dtype, s);
    if (out.status) return out.status;
    // n = T::from_usize(rows); Variable::from(-n)  (cross_entropy.rs:20-21)
    const T neg_n = -(T)n;
    if (ce_single_workgroup(geometry(pred, 1))) {   // a classifier head's batch: probabilities and loss in one launch
        int rc1 = softmax_forward_launch<T, true>(in.ptr, out.ptr, geometry(pred, 1), tin.ptr, nullptr, s,
                                                  static_cast<T *>(loss.ptr), neg_n);
        return rc1 ? rc1 : out.finish();
    }
    Workspace rows((size_t)n * sizeof(T), s);
    if (rows.status) return rows.status;
    T *rowloss = static_cast<T *>(rows.ptr);
    int rc = softmax_forward_launch<T, true>(in.ptr, out.ptr, geometry(pred, 1), tin.ptr, rowloss, s);
    if (rc) return rc;
    if (n <= 65536) {
        ce_finalize_kernel<T><<<1, kBlock, 0, s>>>(rowloss, n, static_cast<T *>(loss.ptr), neg_n);
        ZENU_LAUNCH_CHECK();
    } else {
        Workspace tot(sizeof(T), s);
        if (tot.status) return tot.status;
        const int64_t shape1[1] = {n};
        zenu_tensor_t rv = default_view(rowloss, 1, shape1);
        zenu_tensor_t tv = default_view(tot.ptr, 0, nullptr);
        rc = zenu_hip_sum_all(dtype, tot.ptr, &rv, reinterpret_cast<zenu_stream_t>(s));
        if (!rc) rc = zenu_hip_binary_scalar(ZENU_DIV, dtype, &loss, &tv, (double)neg_n, reinterpret_cast<zenu_stream_t>(s));
        if (rc) return rc;
    }
    return out.finish();
}

template <typename T>
int cross_entropy_backward_t(int dtype, const zenu_tensor_t &gpred, const zenu_tensor_t &prob,
                             const zenu_tensor_t &ans, const zenu_tensor_t *gloss, hipStream_t s,
                             const zenu_tensor_t *gbias = nullptr)
{
    if (num_elm(prob) == 0) return gbias ? ZENU_ERR_SHAPE : ZENU_OK;
    ContigIn<T> yin(prob, dtype, s);
    if (yin.status) return yin.status;
    ContigIn<T> tin(ans, dtype, s);
    if (tin.status) return tin.status;
    ContigOut<T> out(gpred, dtype, s);
    if (out.status) return out.status;
    const T neg_n = -(T)prob.shape[0];
    const T *gout = gloss ? static_cast<const T *>(gloss->ptr) : nullptr;
    T *colsum = gbias ? static_cast<T *>(gbias->ptr) : nullptr;
    int rc = softmax_backward_launch<T, true>(yin.ptr, tin.ptr, out.ptr, geometry(prob, 1), gout, neg_n, s, colsum);
    return rc ? rc : out.finish();
}

template <typename T>
int bias_relu_t(int dtype, const zenu_tensor_t *pre, const zenu_tensor_t &act, const zenu_tensor_t &z,
                const zenu_tensor_t &bias, double alpha, hipStream_t s)
{
    constexpr int VEC = VecOf<T>::N;
    const int64_t n = num_elm(z);
    if (n == 0) return ZENU_OK;
    const int64_t F = bias.shape[0];
    ContigIn<T> zin(z, dtype, s);
    if (zin.status) return zin.status;
    ContigIn<T> bin(bias, dtype, s);
    if (bin.status) return bin.status;
    ContigOut<T> aout(act, dtype, s);
    if (aout.status) return aout.status;
    // `pre` is optional; when absent its ContigOut wraps `act` and is never written or finished
    ContigOut<T> pout(pre ? *pre : act, dtype, s);
    if (pre && pout.status) return pout.status;
    T *pp = pre ? pout.ptr : nullptr;
    const int64_t rows = n / F;
    const bool vec = F % VEC == 0 && aligned16(zin.ptr) && aligned16(bin.ptr) && aligned16(aout.ptr) &&
                     (!pp || aligned16(pp));
    const int64_t packs = vec ? F / VEC : F;
    if (vec && packs % kTileLanes == 0 && rows * (packs / kTileLanes) <= 0x7fffffffLL) {
        const uint32_t tiles = (uint32_t)(packs / kTileLanes);
        const unsigned grid = (unsigned)(rows * tiles);
        const bool nt = n * (int64_t)sizeof(T) * (pp ? 3 : 2) >= kStreamBytes;
        if (nt) bias_relu_tile_kernel<T, VEC, true><<<grid, kTileLanes, 0, s>>>(zin.ptr, bin.ptr, pp, aout.ptr, tiles, (T)alpha);
        else    bias_relu_tile_kernel<T, VEC, false><<<grid, kTileLanes, 0, s>>>(zin.ptr, bin.ptr, pp, aout.ptr, tiles, (T)alpha);
        ZENU_LAUNCH_CHECK();
        int rc2 = aout.finish();
        if (!rc2 && pre) rc2 = pout.finish();
        return rc2;
    }
    int64_t blocks = (rows * packs + kBlock - 1) / kBlock;
    const int64_t cap = (int64_t)device_info().num_cus * 16;
    if (blocks > cap) blocks = cap;
    if (vec) bias_relu_kernel<T, VEC><<<(unsigned)blocks, kBlock, 0, s>>>(zin.ptr, bin.ptr, pp, aout.ptr, rows, packs, (T)alpha);
    else     bias_relu_kernel<T, 1><<<(unsigned)blocks, kBlock, 0, s>>>(zin.ptr, bin.ptr, pp, aout.ptr, rows, packs, (T)alpha);
    ZENU_LAUNCH_CHECK();
    int rc = aout.finish();
    if (!rc && pre) rc = pout.finish();
    return rc;
}

int check_all(const zenu_tensor_t *const *ts, int n)
{
    for (int i = 0; i < n; i++) {
        if (!ts[i]) return ZENU_ERR_ARG;
        int rc = validate_tensor(ts[i]);
        if (rc) return rc;
    }
    return ensure_init();
}

}  // namespace
}  // namespace zenu

using namespace zenu;

extern "C" {

int zenu_hip_softmax(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *src, int axis, zenu_stream_t stream)
{
    const zenu_tensor_t *ts[] = {to, src};
    int rc = check_all(ts, 2);
    if (rc) return rc;
    if (axis < 0 || axis >= src->ndim) return ZENU_ERR_ARG;      // "axis must be less than the number of dimensions"
    if (!same_shape(*to, *src)) return ZENU_ERR_SHAPE;           // "softmax shape mismatch"
    if (dtype == ZENU_F32) return softmax_t<float>(dtype, *to, *src, axis, as_stream(stream));
    if (dtype == ZENU_F64) return softmax_t<double>(dtype, *to, *src, axis, as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_softmax_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *y, const zenu_tensor_t *gy,
                              int axis, zenu_stream_t stream)
{
    const zenu_tensor_t *ts[] = {gx, y, gy};
    int rc = check_all(ts, 3);
    if (rc) return rc;
    if (axis < 0 || axis >= y->ndim) return ZENU_ERR_ARG;
    if (!same_shape(*gx, *y) || !same_shape(*gy, *y)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) return softmax_backward_t<float>(dtype, *gx, *y, *gy, axis, as_stream(stream));
    if (dtype == ZENU_F64) return softmax_backward_t<double>(dtype, *gx, *y, *gy, axis, as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_softmax_cross_entropy(int dtype, const zenu_tensor_t *loss, const zenu_tensor_t *prob,
                                   const zenu_tensor_t *pred, const zenu_tensor_t *ans, zenu_stream_t stream)
{
    const zenu_tensor_t *ts[] = {loss, prob, pred, ans};
    int rc = check_all(ts, 4);
    if (rc) return rc;
    if (pred->ndim != 2 || loss->ndim != 0) return ZENU_ERR_SHAPE;   // softmax(pred, 1), sum_to(.., [])
    if (!same_shape(*prob, *pred) || !same_shape(*ans, *pred)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) return cross_entropy_t<float>(dtype, *loss, *prob, *pred, *ans, as_stream(stream));
    if (dtype == ZENU_F64) return cross_entropy_t<double>(dtype, *loss, *prob, *pred, *ans, as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_softmax_cross_entropy_backward(int dtype, const zenu_tensor_t *gpred, const zenu_tensor_t *prob,
                                            const zenu_tensor_t *ans, const zenu_tensor_t *gloss,
                                            zenu_stream_t stream)
{
    const zenu_tensor_t *ts[] = {gpred, prob, ans};
    int rc = check_all(ts, 3);
    if (rc) return rc;
    if (gloss && (validate_tensor(gloss) || gloss->ndim != 0)) return ZENU_ERR_SHAPE;
    if (prob->ndim != 2) return ZENU_ERR_SHAPE;
    if (!same_shape(*gpred, *prob) || !same_shape(*ans, *prob)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) return cross_entropy_backward_t<float>(dtype, *gpred, *prob, *ans, gloss, as_stream(stream));
    if (dtype == ZENU_F64) return cross_entropy_backward_t<double>(dtype, *gpred, *prob, *ans, gloss, as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_softmax_cross_entropy_backward_bias_grad(int dtype, const zenu_tensor_t *gpred, const zenu_tensor_t *gbias,
                                                      const zenu_tensor_t *prob, const zenu_tensor_t *ans,
                                                      const zenu_tensor_t *gloss, zenu_stream_t stream)
{
    const zenu_tensor_t *ts[] = {gpred, gbias, prob, ans};
    int rc = check_all(ts, 4);
    if (rc) return rc;
    if (gloss && (validate_tensor(gloss) || gloss->ndim != 0)) return ZENU_ERR_SHAPE;
    if (prob->ndim != 2) return ZENU_ERR_SHAPE;
    if (!same_shape(*gpred, *prob) || !same_shape(*ans, *prob)) return ZENU_ERR_SHAPE;
    if (gbias->ndim < 1 || gbias->shape[gbias->ndim - 1] != prob->shape[1] || num_elm(*gbias) != prob->shape[1])
        return ZENU_ERR_SHAPE;
    if (dtype != ZENU_F32 && dtype != ZENU_F64) return ZENU_ERR_ARG;
    const size_t esz = dtype == ZENU_F32 ? 4 : 8;
    const size_t gb_bytes = (size_t)num_elm(*gbias) * esz;
    if (view_overlaps(*gpred, esz, gbias->ptr, gb_bytes) || view_overlaps(*prob, esz, gbias->ptr, gb_bytes) ||
        view_overlaps(*ans, esz, gbias->ptr, gb_bytes))
        return ZENU_ERR_ARG;
    // a classifier head's batch (every line in one workgroup, at most 16 classes): gradient and its column
    // sums in one launch; anything else is the two calls it stands for
    if (prob->shape[0] <= kBlock && prob->shape[1] <= kLineRegs && is_default_stride_strict(*gbias)) {
        rc = dtype == ZENU_F32
                 ? cross_entropy_backward_t<float>(dtype, *gpred, *prob, *ans, gloss, as_stream(stream), gbias)
                 : cross_entropy_backward_t<double>(dtype, *gpred, *prob, *ans, gloss, as_stream(stream), gbias);
        if (rc != ZENU_ERR_UNSUPPORTED) return rc;
    }
    rc = zenu_hip_softmax_cross_entropy_backward(dtype, gpred, prob, ans, gloss, stream);
    if (rc) return rc;
    return zenu_hip_sum_to(dtype, gbias, gpred, stream);
}

int zenu_hip_bias_add_relu(int dtype, const zenu_tensor_t *pre, const zenu_tensor_t *act, const zenu_tensor_t *z,
                           const zenu_tensor_t *bias, double alpha, zenu_stream_t stream)
{
    const zenu_tensor_t *ts[] = {act, z, bias};
    int rc = check_all(ts, 3);
    if (rc) return rc;
    if (pre && validate_tensor(pre)) return ZENU_ERR_ARG;
    if (z->ndim < 1 || bias->ndim != 1 || bias->shape[0] != z->shape[z->ndim - 1]) return ZENU_ERR_SHAPE;
    if (!same_shape(*act, *z) || (pre && !same_shape(*pre, *z))) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) return bias_relu_t<float>(dtype, pre, *act, *z, *bias, alpha, as_stream(stream));
    if (dtype == ZENU_F64) return bias_relu_t<double>(dtype, pre, *act, *z, *bias, alpha, as_stream(stream));
    return ZENU_ERR_ARG;
}

}  // extern "C"
