/*
 * zenu_oracle.c -- CPU restatement of ZeNu's Cpu device path.
 * TEST INFRASTRUCTURE ONLY: the checker for the HIP kernels and the CPU baseline of the
 * benchmark.  See zenu_oracle.h for the reference files each part follows.
 *
 * Build: gcc -O2 -fno-fast-math -ffp-contract=off (no FMA fusion, IEEE semantics), one thread.
 *
 * Pinning status of each function group (how the restatement is checked without running the
 * reference, which is Rust and cannot be built in this environment):
 *   binary / scalar / broadcast / strided ops : reference test vectors
 *       (basic_operations.rs:649-1335, with_clousers.rs:356-508) + brute-force N-d loops
 *   unary exp/log/tanh/sqrt/abs/sin..cosh, pow : reference literal tables
 *       (zenu-cuda/src/kernel/mod.rs:1015-1241, basic_operations.rs:1341-1451) + same libm symbols
 *   relu / relu_backward_mask : relu.rs:255-296, zenu-cuda/src/kernel/activation.rs:88-147
 *   sigmoid : zenu-autograd/src/activation/sigmoid.rs:26-66
 *   sum / sum_to : sum.rs:109-245 + f64 brute force
 *   max_idx / max_axis / max_axis_idx_ravel : max.rs:157-844 + brute force incl. ties / NaN
 *   copy_from : copy_from.rs:285-398, to_default_stride.rs:28-89
 *   SGD / Adam / AdamW : zenu-optimizer/tests/net_test.rs:107-232 (via a tiny Linear+MSE net
 *       restated in the test) + closed-form invariants
 *   asum : asum.rs:78-120 for small exact integers; accumulation order of OpenBLAS
 *       s/dasum is PARITY UNPINNED (compared with a tolerance)
 */
#include "zenu_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

static uint64_t g_leaf_calls = 0;

uint64_t zo_leaf_calls(void) { return g_leaf_calls; }
void zo_reset_leaf_calls(void) { g_leaf_calls = 0; }

/* dim/mod.rs:70-92 */
void zo_default_stride(int ndim, const int64_t *shape, int64_t *stride)
{
    if (ndim == 0) return;
    stride[ndim - 1] = 1;
    for (int i = ndim - 2; i >= 0; i--) stride[i] = stride[i + 1] * shape[i + 1];
}

static int64_t zo_num_elm(const zo_view *v)
{
    int64_t n = 1;
    for (int i = 0; i < v->ndim; i++) n *= v->shape[i];
    return n;
}

/* dim/mod.rs:40-42 */
static int zo_is_scalar(const zo_view *v) { return v->ndim == 0 || zo_num_elm(v) == 1; }

static int64_t zo_last_stride(const zo_view *v) { return v->ndim ? v->stride[v->ndim - 1] : 1; }

static int zo_is_strict_default_stride(const zo_view *v)
{
    int64_t d[ZO_MAX_DIM];
    zo_default_stride(v->ndim, v->shape, d);
    for (int i = 0; i < v->ndim; i++)
        if (d[i] != v->stride[i]) return 0;
    return 1;
}

/* shape_stride.rs:116-121: every 1-D view counts as default stride whatever its stride */
int zo_is_default_stride(const zo_view *v)
{
    if (v->ndim == 1) return 1;
    return zo_is_strict_default_stride(v);
}

/* shape_stride.rs:65-83 */
int zo_is_contiguous(const zo_view *v)
{
    int nd = v->ndim;
    if (nd == 0) return 1;
    int order[ZO_MAX_DIM];
    for (int i = 0; i < nd; i++) order[i] = i;
    /* stable sort by stride, descending */
    for (int i = 1; i < nd; i++) {
        int o = order[i], j = i - 1;
        while (j >= 0 && v->stride[order[j]] < v->stride[o]) { order[j + 1] = order[j]; j--; }
        order[j + 1] = o;
    }
    int64_t sshape[ZO_MAX_DIM], sstride[ZO_MAX_DIM], d[ZO_MAX_DIM];
    for (int i = 0; i < nd; i++) { sshape[i] = v->shape[order[i]]; sstride[i] = v->stride[order[i]]; }
    zo_default_stride(nd, sshape, d);
    if (sstride[0] == 0) return 0; /* the reference divides by zero here */
    int64_t n = d[0] / sstride[0];
    if (d[0] % sstride[0] != 0) return 0;
    for (int i = 0; i < nd; i++)
        if (d[i] * n != sstride[i]) return 0;
    return 1;
}

static int zo_dims_equal(int na, const int64_t *a, int nb, const int64_t *b)
{
    if (na != nb) return 0;
    for (int i = 0; i < na; i++)
        if (a[i] != b[i]) return 0;
    return 1;
}

static int zo_same_shape(const zo_view *a, const zo_view *b)
{
    return zo_dims_equal(a->ndim, a->shape, b->ndim, b->shape);
}

/* dim_dyn.rs:119-130 */
static int zo_dim_is_include(int ns, const int64_t *s, int no, const int64_t *o)
{
    if (ns < no) return zo_dim_is_include(no, o, ns, s);
    for (int i = 0; i < no; i++)
        if (s[ns - 1 - i] != o[no - 1 - i]) return 0;
    return 1;
}

/* dim_dyn.rs:137-148 (the caller guarantees ns >= no; the reference asserts it) */
static int zo_dim_is_include_broadcast(int ns, const int64_t *s, int no, const int64_t *o)
{
    if (ns < no) return 0;
    for (int i = 0; i < no; i++) {
        if (s[ns - 1 - i] == o[no - 1 - i] || o[no - 1 - i] == 1) continue;
        return 0;
    }
    return 1;
}

/* dim_dyn.rs:24-47 */
int zo_larger_shape(int nx, const int64_t *x, int ny, const int64_t *y)
{
    if (nx < ny) return zo_dim_is_include(ny, y, nx, x) ? 1 : -ZO_ERR_SHAPE;
    if (nx > ny) return zo_dim_is_include(nx, x, ny, y) ? 0 : -ZO_ERR_SHAPE;
    if (zo_dim_is_include_broadcast(nx, x, ny, y)) return 0;
    if (zo_dim_is_include_broadcast(ny, y, nx, x)) return 1;
    return -ZO_ERR_SHAPE;
}

/* ---- float instance ---- */
#define T float
#define S f32
#define ZO_EXP_FN expf
#define ZO_LOG_FN logf
#define ZO_TANH_FN tanhf
#define ZO_SQRT_FN sqrtf
#define ZO_FABS_FN fabsf
#define ZO_SIN_FN sinf
#define ZO_COS_FN cosf
#define ZO_TAN_FN tanf
#define ZO_ASIN_FN asinf
#define ZO_ACOS_FN acosf
#define ZO_ATAN_FN atanf
#define ZO_SINH_FN sinhf
#define ZO_COSH_FN coshf
#define ZO_POW_FN powf
#include "zenu_oracle_impl.inc"
#undef T
#undef S
#undef ZO_EXP_FN
#undef ZO_LOG_FN
#undef ZO_TANH_FN
#undef ZO_SQRT_FN
#undef ZO_FABS_FN
#undef ZO_SIN_FN
#undef ZO_COS_FN
#undef ZO_TAN_FN
#undef ZO_ASIN_FN
#undef ZO_ACOS_FN
#undef ZO_ATAN_FN
#undef ZO_SINH_FN
#undef ZO_COSH_FN
#undef ZO_POW_FN

/* ---- double instance ---- */
#define T double
#define S f64
#define ZO_EXP_FN exp
#define ZO_LOG_FN log
#define ZO_TANH_FN tanh
#define ZO_SQRT_FN sqrt
#define ZO_FABS_FN fabs
#define ZO_SIN_FN sin
#define ZO_COS_FN cos
#define ZO_TAN_FN tan
#define ZO_ASIN_FN asin
#define ZO_ACOS_FN acos
#define ZO_ATAN_FN atan
#define ZO_SINH_FN sinh
#define ZO_COSH_FN cosh
#define ZO_POW_FN pow
#include "zenu_oracle_impl.inc"

/* ------------------------------------------------------------------ */
/* Every f32 bit pattern of a range through one unary function, folded   */
/* into a 64-bit sum per block of patterns.  The library computes the    */
/* same sums on the device (zenu_hip_unary_range_hash); equal sums mean  */
/* equal results on every argument of the block, with nothing copied.    */
/* The functions are the libm calls of zo_unary_fn_f32 and the sigmoid   */
/* composite of zo_sigmoid_f32 (x*half, tanh, half*t, half+u, each        */
/* rounded to f32).  Threads only split the range.                       */
/* ------------------------------------------------------------------ */
#include <pthread.h>

/* one term: the argument's and the result's bits through the finalizer of splitmix64; every NaN counts as one value */
uint64_t zo_range_hash_term(uint32_t arg_bits, uint32_t res_bits)
{
    if ((res_bits & 0x7fffffffu) > 0x7f800000u) res_bits = 0x7fc00000u;
    uint64_t z = ((uint64_t)arg_bits << 32) | res_bits;
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

static inline float zo_range_fn(int fn, float x)
{
    if (fn == ZO_SIGMOID_COMPOSITE) {
        const float half = 1.0f / (1.0f + 1.0f);
        const float t1 = x * half;
        const float t2 = tanhf(t1);
        const float t3 = half * t2;
        return half + t3;
    }
    return zo_unary_fn_f32(fn, x);
}

static inline uint64_t zo_mix64(uint64_t z)
{
    z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
    z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
    return z ^ (z >> 31);
}

/* f64 argument number i: high word i * step + offset, a pseudo-random low word from i and salt */
uint64_t zo_range_arg_f64(uint64_t i, uint32_t step, uint32_t offset, uint64_t salt)
{
    const uint64_t hi = (uint32_t)(i * step + offset);
    const uint64_t lo = (uint32_t)(((i + salt) * 0x9E3779B97F4A7C15ull) >> 29);
    return (hi << 32) | lo;
}

static inline double zo_range_fn_f64(int fn, double x)
{
    if (fn == ZO_SIGMOID_COMPOSITE) {
        const double half = 1.0 / (1.0 + 1.0);
        const double t1 = x * half;
        const double t2 = tanh(t1);
        const double t3 = half * t2;
        return half + t3;
    }
    return zo_unary_fn_f64(fn, x);
}

/* kind 0: f32 unary (fn); kind 1: f32 powf with `exponent`; kind 2: f64 unary (fn) on zo_range_arg_f64; kind 3: f64 pow with `exponent64` */
typedef struct {
    int kind, fn, block_log2;
    float exponent;
    double exponent64;
    uint32_t step, offset;
    uint64_t salt;
    uint64_t first_block, n_blocks, first;
    uint64_t *sums;
} zo_range_job;

static void *zo_range_worker(void *arg)
{
    const zo_range_job *j = (const zo_range_job *)arg;
    const uint64_t per = 1ull << j->block_log2;
    for (uint64_t b = j->first_block; b < j->first_block + j->n_blocks; b++) {
        uint64_t sum = 0;
        const uint64_t start = j->first + b * per;
        if (j->kind == 2 || j->kind == 3) {
            for (uint64_t i = 0; i < per; i++) {
                const uint64_t bits = zo_range_arg_f64(start + i, j->step, j->offset, j->salt);
                double x, y;
                uint64_t rb;
                memcpy(&x, &bits, 8);
                y = j->kind == 3 ? pow(x, j->exponent64) : zo_range_fn_f64(j->fn, x);
                memcpy(&rb, &y, 8);
                if ((rb & 0x7fffffffffffffffull) > 0x7ff0000000000000ull) rb = 0x7ff8000000000000ull;
                sum += zo_mix64(zo_mix64(bits) + rb);
            }
        } else {
            for (uint64_t i = 0; i < per; i++) {
                const uint32_t bits = (uint32_t)(start + i);
                float x, y;
                uint32_t rb;
                memcpy(&x, &bits, 4);
                y = j->kind == 1 ? powf(x, j->exponent) : zo_range_fn(j->fn, x);
                memcpy(&rb, &y, 4);
                sum += zo_range_hash_term(bits, rb);
            }
        }
        j->sums[b] = sum;
    }
    return NULL;
}

/* sums[b] for the patterns first + b * 2^block_log2 ... of `count` patterns (a multiple of the block size) */
static int zo_range_hash_run(zo_range_job proto, uint64_t first, uint64_t count, int block_log2, uint64_t *sums, int nthreads)
{
    if (block_log2 < 0 || block_log2 > 32 || (count & ((1ull << block_log2) - 1)) || first + count > (1ull << 32))
        return ZO_ERR_ARG;
    if (proto.kind != 1 && (proto.fn < ZO_EXP || proto.fn > ZO_SIGMOID_COMPOSITE)) return ZO_ERR_ARG;
    const uint64_t blocks = count >> block_log2;
    if (nthreads < 1) nthreads = 1;
    if (nthreads > 64) nthreads = 64;
    if ((uint64_t)nthreads > blocks) nthreads = (int)(blocks ? blocks : 1);
    pthread_t th[64];
    zo_range_job jobs[64];
    uint64_t next = 0;
    for (int t = 0; t < nthreads; t++) {
        const uint64_t share = blocks / (uint64_t)nthreads + ((uint64_t)t < blocks % (uint64_t)nthreads ? 1 : 0);
        jobs[t] = proto;
        jobs[t].block_log2 = block_log2;
        jobs[t].first = first;
        jobs[t].first_block = next;
        jobs[t].n_blocks = share;
        jobs[t].sums = sums;
        next += share;
    }
    int started = 1;
    for (; started < nthreads; started++)
        if (pthread_create(&th[started], NULL, zo_range_worker, &jobs[started])) break;
    zo_range_worker(&jobs[0]);
    for (int t = started; t < nthreads; t++) zo_range_worker(&jobs[t]);   /* threads that could not be started: done here */
    for (int t = 1; t < started; t++) pthread_join(th[t], NULL);
    return ZO_OK;
}

int zo_unary_range_hash_f32(int fn, uint64_t first, uint64_t count, int block_log2, uint64_t *sums, int nthreads)
{
    zo_range_job j;
    memset(&j, 0, sizeof j);
    j.kind = 0;
    j.fn = fn;
    return zo_range_hash_run(j, first, count, block_log2, sums, nthreads);
}

/* the same for powf(x, exponent) over the f32 bases x */
int zo_powf_range_hash_f32(float exponent, uint64_t first, uint64_t count, int block_log2, uint64_t *sums, int nthreads)
{
    zo_range_job j;
    memset(&j, 0, sizeof j);
    j.kind = 1;
    j.exponent = exponent;
    return zo_range_hash_run(j, first, count, block_log2, sums, nthreads);
}

/* f64: argument number i of [first, first + count) is zo_range_arg_f64(i, step, offset, salt); the term is
 * mix64(mix64(argument bits) + result bits), every NaN result counted as 0x7ff8000000000000 */
int zo_unary_range_hash_f64(int fn, uint64_t first, uint64_t count, int block_log2, uint32_t step, uint32_t offset,
                            uint64_t salt, uint64_t *sums, int nthreads)
{
    zo_range_job j;
    memset(&j, 0, sizeof j);
    if (step == 0) return ZO_ERR_ARG;
    j.kind = 2;
    j.fn = fn;
    j.step = step;
    j.offset = offset;
    j.salt = salt;
    return zo_range_hash_run(j, first, count, block_log2, sums, nthreads);
}

/* the same for pow(x, exponent) over the sampled f64 bases x */
int zo_powf_range_hash_f64(double exponent, uint64_t first, uint64_t count, int block_log2, uint32_t step, uint32_t offset,
                           uint64_t salt, uint64_t *sums, int nthreads)
{
    zo_range_job j;
    memset(&j, 0, sizeof j);
    if (step == 0) return ZO_ERR_ARG;
    j.kind = 3;
    j.exponent64 = exponent;
    j.step = step;
    j.offset = offset;
    j.salt = salt;
    return zo_range_hash_run(j, first, count, block_log2, sums, nthreads);
}

