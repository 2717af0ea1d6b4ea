/*
 * zenu_oracle.h -- CPU restatement of ZeNu's Cpu device path (TEST INFRASTRUCTURE ONLY).
 *
 * This library is the checker for the HIP kernels: tests, the smoke check and the
 * cpu_baseline leg of the benchmark may link or load it.  Nothing in the product
 * (the HIP library or the host layer above it) may call into it.
 *
 * It restates, single-threaded and in the reference's evaluation order, the
 * algorithms of the reference's CPU path:
 *   - the 1-D strided leaf loops of the device traits
 *       zenu-matrix/src/operation/basic_operations.rs:91-182,397-421
 *       zenu-matrix/src/operation/relu.rs:31-91
 *       zenu-matrix/src/operation/max.rs:19-34
 *   - the host-side N-d -> 1-D decomposition (one leaf call per row / slice)
 *       zenu-matrix/src/with_clousers.rs:9-242
 *       zenu-matrix/src/operation/basic_operations.rs:278-381,512-575
 *       zenu-matrix/src/operation/relu.rs:169-242
 *   - sum / sum_to               zenu-matrix/src/operation/sum.rs:9-94
 *   - max_idx / max_axis / max_axis_idx_ravel
 *                                zenu-matrix/src/operation/max.rs:43-135
 *   - asum (plain loop; the reference calls OpenBLAS sasum/dasum whose
 *     accumulation order is not specified -> "parity unpinned", compared with
 *     a tolerance)               zenu-matrix/src/operation/asum.rs:49-68
 *   - copy_from / to_default_stride
 *                                zenu-matrix/src/operation/copy_from.rs:211-267
 *   - sigmoid composite          zenu-autograd/src/activation/sigmoid.rs:7-15
 *   - SGD / Adam / AdamW         zenu-optimizer/src/{sgd.rs:20-31,adam.rs:19-59,adamw.rs:20-70}
 *   - clip / clip masks          zenu-matrix/src/operation/clip.rs:39-110,205-318
 *   - broadcast                  zenu-matrix/src/operation/broadcast.rs:11-43
 * The chains built from these (softmax_assign, SoftMax::backward, cross_entropy and its
 * backward, bias add + relu) are composed op by op in tests/cpu_matrix.py.
 *
 * Pinned by the reference's own known-answer tests, restated in tests/ref_cases.py and
 * tests/test_optimizer_net.py and run against this library by tests/test_oracle_ref_cases.py
 * (binary/scalar/broadcast/strided ops, unary tables, relu, sigmoid, sum, sum_to, max*,
 * copy, clip, broadcast, softmax, cross-entropy, the optimizers' net_test.rs literals).
 * Parity unpinned: the accumulation order of asum (OpenBLAS) only.
 *
 * exp/log/tanh/pow call the host libm (expf/logf/tanhf/powf, exp/log/tanh/pow):
 * the same symbols Rust's f32::exp/ln/tanh/powf lower to.
 *
 * Every entry exists for float (suffix _f32) and double (suffix _f64).
 * Strides are in ELEMENTS.  A view's ptr already includes its offset.
 * Functions returning int return 0 on success and a ZO_ERR_* code where the
 * reference would panic (shape / rank / axis errors).
 */
#ifndef ZENU_ORACLE_H
#define ZENU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ZO_MAX_DIM 6

typedef struct zo_view {
    void   *ptr;                 /* base pointer + offset, element type given by the suffix */
    int32_t ndim;                /* 0..6 (0 = scalar) */
    int32_t reserved;
    int64_t shape[ZO_MAX_DIM];
    int64_t stride[ZO_MAX_DIM];  /* in elements */
} zo_view;

enum { ZO_OK = 0, ZO_ERR_RANK = 1, ZO_ERR_SHAPE = 2, ZO_ERR_AXIS = 3, ZO_ERR_ARG = 4 };
enum { ZO_ADD = 0, ZO_SUB = 1, ZO_MUL = 2, ZO_DIV = 3 };
enum {
    ZO_EXP = 0, ZO_LOG = 1, ZO_TANH = 2, ZO_SQRT = 3, ZO_ABS = 4,
    ZO_SIN = 5, ZO_COS = 6, ZO_TAN = 7, ZO_ASIN = 8, ZO_ACOS = 9, ZO_ATAN = 10,
    ZO_SINH = 11, ZO_COSH = 12
};
/* for zo_unary_range_hash_f32 only: the sigmoid composite of zo_sigmoid_f32 as a function of one argument */
enum { ZO_SIGMOID_COMPOSITE = 13 };

/* number of leaf (device-trait) calls issued since the last reset: mirrors the
 * call-counting tests of zenu-matrix/src/with_clousers.rs:356-379 */
uint64_t zo_leaf_calls(void);
void     zo_reset_leaf_calls(void);

/* shape helpers shared by both dtypes */
void zo_default_stride(int ndim, const int64_t *shape, int64_t *stride);
int  zo_is_default_stride(const zo_view *v);
int  zo_is_contiguous(const zo_view *v);
/* larger_shape (dim_dyn.rs:24-58): writes the broadcast result shape; returns
 * 0 if x is the larger, 1 if y is, <0 (-ZO_ERR_SHAPE) where the reference panics */
int  zo_larger_shape(int nx, const int64_t *x, int ny, const int64_t *y);

#define ZO_DECLARE(T, S)                                                                           \
    /* ---- device-trait leaves (1-D strided loops) ---- */                                        \
    void zo_array_array_##S(int op, T *to, const T *lhs, const T *rhs, size_t n, size_t st,       \
                            size_t sl, size_t sr);                                                 \
    void zo_array_assign_##S(int op, T *to, const T *rhs, size_t n, size_t st, size_t sr);        \
    void zo_scalar_##S(int op, T *to, const T *lhs, T rhs, size_t n, size_t st, size_t sl);       \
    void zo_scalar_assign_##S(int op, T *to, T rhs, size_t n, size_t st);                         \
    void zo_scalar_ptr_##S(int op, T *to, const T *lhs, const T *scalar, size_t st, size_t sl,    \
                           size_t n);                                                              \
    void zo_scalar_assign_ptr_##S(int op, T *to, const T *scalar, size_t n, size_t st);           \
    void zo_unary_leaf_##S(int fn, T *to, const T *other, size_t n, size_t st, size_t so);        \
    void zo_unary_assign_leaf_##S(int fn, T *to, size_t n, size_t st);                            \
    void zo_pow_leaf_##S(T *to, const T *other, T scalar, size_t n, size_t st, size_t so);        \
    void zo_relu_leaf_##S(const T *input, T *output, T alpha, size_t n, size_t si, size_t so);    \
    void zo_relu_backward_mask_leaf_##S(const T *input, T *mask, T alpha, size_t n, size_t si,    \
                                        size_t sm);                                                \
    size_t zo_max_idx_leaf_##S(const T *input, size_t size, size_t stride);                       \
    T    zo_asum_leaf_##S(size_t n, const T *x, size_t incx);                                     \
    /* ---- Matrix-level ops (reference-shaped decomposition) ---- */                              \
    int zo_binary_array_##S(int op, const zo_view *to, const zo_view *lhs, const zo_view *rhs);   \
    int zo_binary_assign_##S(int op, const zo_view *to, const zo_view *rhs);                      \
    int zo_binary_scalar_##S(int op, const zo_view *to, const zo_view *other, T scalar);          \
    int zo_binary_scalar_assign_##S(int op, const zo_view *to, T scalar);                         \
    int zo_unary_##S(int fn, const zo_view *to, const zo_view *other);                            \
    int zo_unary_assign_##S(int fn, const zo_view *to);                                           \
    int zo_powf_##S(const zo_view *to, const zo_view *other, T scalar);                           \
    int zo_relu_##S(const zo_view *to, const zo_view *other, T alpha);                            \
    int zo_relu_backward_mask_##S(const zo_view *to, const zo_view *other, T alpha);              \
    /* zenu-matrix/src/operation/broadcast.rs:11-43 */                                             \
    int zo_broadcast_##S(const zo_view *to, const zo_view *source);                               \
    /* zenu-matrix/src/operation/clip.rs:39-110, 205-318 */                                        \
    int zo_clip_##S(const zo_view *to, const zo_view *other, T min, T max);                       \
    int zo_clip_backward_mask_##S(const zo_view *mask, const zo_view *other, T min, T max);       \
    int zo_sigmoid_##S(const zo_view *to, const zo_view *x);                                      \
    int zo_copy_from_##S(const zo_view *to, const zo_view *src);                                  \
    /* out: caller-allocated default-stride buffer with shape = src.shape minus axis */           \
    int zo_sum_##S(const zo_view *src, int axis, T *out);                                         \
    int zo_sum_to_##S(const zo_view *src, const zo_view *target);                                 \
    /* idx_out: N-d index (src.ndim entries) of the first maximum in row-major order */           \
    int zo_max_idx_##S(const zo_view *src, int64_t *idx_out);                                     \
    int zo_max_item_##S(const zo_view *src, T *out);                                              \
    int zo_max_axis_##S(const zo_view *src, int axis, T *out);                                    \
    int zo_max_axis_idx_ravel_##S(const zo_view *src, int axis, int64_t *out);                    \
    T   zo_asum_##S(const zo_view *src);                                                          \
    /* ---- optimizers on one parameter tensor (flat, n elements) ---- */                          \
    void zo_sgd_update_##S(T *p, const T *g, size_t n, T lr);                                     \
    /* step = value of the step counter AFTER the increment (adam.rs:21-22) */                    \
    void zo_adam_update_##S(T *p, const T *g, T *m, T *v, size_t n, T lr, T beta1, T beta2,       \
                            T eps, T step);                                                        \
    void zo_adamw_update_##S(T *p, const T *g, T *m, T *v, size_t n, T lr, T beta1, T beta2,      \
                             T eps, T weight_decay, int is_weight, T step);                        \
    /* fused single-pass loops with identical per-element arithmetic (plain-loop CPU figure) */   \
    void zo_adam_update_fused_##S(T *p, const T *g, T *m, T *v, size_t n, T lr, T beta1,          \
                                  T beta2, T eps, T weight_decay, int is_weight, int adamw,       \
                                  T step);

ZO_DECLARE(float, f32)
ZO_DECLARE(double, f64)

/* Every f32 bit pattern of [first, first + count) through unary function `fn` (ZO_EXP ... ZO_COSH, or
 * ZO_SIGMOID_COMPOSITE), folded into one 64-bit sum per block of 2^block_log2 patterns:
 * sums[b] = sum over the block of zo_range_hash_term(argument bits, result bits) mod 2^64.  The HIP
 * library computes the same sums on the device, so that every argument can be compared without
 * copying results.  `nthreads` threads split the blocks (the functions themselves stay the plain
 * libm calls of the one-thread path). */
uint64_t zo_range_hash_term(uint32_t arg_bits, uint32_t res_bits);
int zo_unary_range_hash_f32(int fn, uint64_t first, uint64_t count, int block_log2, uint64_t *sums, int nthreads);
/* the same for powf(x, exponent) over the f32 bases, and for the f64 functions on sampled arguments:
 * argument number i is zo_range_arg_f64(i, step, offset, salt) (high word i * step + offset, a
 * pseudo-random low word), the term mix64(mix64(argument bits) + result bits) with mix64 the finalizer of
 * splitmix64 and every NaN result counted as 0x7ff8000000000000 */
int zo_powf_range_hash_f32(float exponent, uint64_t first, uint64_t count, int block_log2, uint64_t *sums, int nthreads);
uint64_t zo_range_arg_f64(uint64_t i, uint32_t step, uint32_t offset, uint64_t salt);
int zo_unary_range_hash_f64(int fn, uint64_t first, uint64_t count, int block_log2, uint32_t step, uint32_t offset,
                            uint64_t salt, uint64_t *sums, int nthreads);
int zo_powf_range_hash_f64(double exponent, uint64_t first, uint64_t count, int block_log2, uint32_t step, uint32_t offset,
                           uint64_t salt, uint64_t *sums, int nthreads);

#ifdef __cplusplus
}
#endif
#endif /* ZENU_ORACLE_H */
