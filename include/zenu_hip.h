/*
 * zenu_hip.h -- C ABI of the MI355X (gfx950) device tensor-kernel layer for ZeNu.
 *
 * This is the boundary a `Hip` device of zenu-matrix binds to, in place of the
 * bindgen output over zenu-cuda-kernel-sys/kernel/kernel.h and of the cudart
 * wrappers in zenu-cuda/src/runtime/mod.rs.  Plain pointers and sizes only.
 *
 * Conventions
 *   - every pointer named *_dev / inside a zenu_tensor_t is DEVICE memory;
 *   - strides are in ELEMENTS; a tensor's ptr already includes its offset
 *     (Matrix::as_ptr, zenu-matrix/src/matrix.rs:288-290);
 *   - at most 6 dimensions (zenu-matrix/src/dim/dim_dyn.rs:10-13,75);
 *   - `stream` is a hipStream_t passed as void*; NULL = the HIP null stream;
 *     all launches are asynchronous on that stream unless stated otherwise;
 *   - every function returns ZENU_OK (0) or an error code; nothing aborts.  Where the
 *     reference panics (shape / rank / axis mismatch) the code is ZENU_ERR_SHAPE,
 *     ZENU_ERR_RANK or ZENU_ERR_AXIS and nothing is launched.
 *   - an input may be the output's own view (the *_assign forms: same pointer, same strides);
 *     an input that shares memory with an output in any other way (shifted, transposed or
 *     broadcast views of it; a reduction's result inside its source; optimizer arrays that
 *     overlap) is refused with ZENU_ERR_ARG and nothing is launched.  ZeNu's `&mut` outputs
 *     cannot alias their `&` inputs, so no call the reference can make is affected.
 */
#ifndef ZENU_HIP_H
#define ZENU_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ZENU_MAX_DIM 6

typedef enum {
    ZENU_OK = 0,
    ZENU_ERR_RANK = 1,        /* "The rank of the matrix is different."      */
    ZENU_ERR_SHAPE = 2,       /* shapes not broadcast-compatible / mismatch  */
    ZENU_ERR_AXIS = 3,        /* "Invalid axis" / "Axis out of bounds"       */
    ZENU_ERR_ARG = 4,         /* null pointer, bad enum, ndim > 6, negative size */
    ZENU_ERR_HIP = 5,         /* a HIP runtime call failed: see zenu_hip_last_hip_error */
    ZENU_ERR_OOM = 6,         /* device allocation failed even after trimming the cache */
    ZENU_ERR_UNSUPPORTED = 7, /* valid request this build has no kernel for  */
    ZENU_ERR_NOT_OWNED = 8,   /* zenu_hip_free: pointer unknown to the pool (MemPoolFreeError) */
    ZENU_ERR_NOT_INIT = 9,    /* an entry point that may not allocate was called before zenu_hip_init */
    ZENU_ERR_SCRATCH_LIMIT = 10 /* zenu_hip_sum_axis_noalloc: the request needs more than its static scratch */
} zenu_status_t;

typedef enum { ZENU_F32 = 0, ZENU_F64 = 1 } zenu_dtype_t;

typedef enum { ZENU_ADD = 0, ZENU_SUB = 1, ZENU_MUL = 2, ZENU_DIV = 3 } zenu_binop_t;

typedef enum {
    ZENU_EXP = 0, ZENU_LOG = 1, ZENU_TANH = 2, ZENU_SQRT = 3, ZENU_ABS = 4,
    ZENU_SIN = 5, ZENU_COS = 6, ZENU_TAN = 7, ZENU_ASIN = 8, ZENU_ACOS = 9, ZENU_ATAN = 10,
    ZENU_SINH = 11, ZENU_COSH = 12,
    ZENU_SIGMOID = 13, /* 0.5 + 0.5*tanh(0.5*x), zenu-autograd/src/activation/sigmoid.rs:7-15 */
    /* No counterpart in the reference.  ZENU_TANH returns the bits of the host library's tanhf (what
     * ZeNu's Cpu device returns) and is bound by arithmetic, not memory.  ZENU_TANH_ULP2 is for
     * callers that accept the usual tolerance instead: f32 tanh evaluated in f64 and rounded once,
     * at most 2 units in the last place from ZENU_TANH on every one of the 2^32 arguments, and
     * bound by memory.  For f64 it is ZENU_TANH. */
    ZENU_TANH_ULP2 = 14
} zenu_unop_t;

/* A strided view: Matrix<_, DimDyn, D> flattened (zenu-matrix/src/matrix.rs:224-233). */
typedef struct zenu_tensor {
    void   *ptr;
    int32_t ndim;
    int32_t reserved;
    int64_t shape[ZENU_MAX_DIM];
    int64_t stride[ZENU_MAX_DIM];
} zenu_tensor_t;

typedef void *zenu_stream_t;

/* ------------------------------------------------------------------------- */
/* Runtime: replaces zenu-cuda/src/runtime/mod.rs and zenu-cuda/src/lib.rs    */
/* ------------------------------------------------------------------------- */

/* Select the device and create the library state (allocator, default stream).
 * Idempotent.  zenu-cuda/src/lib.rs:18-25,60-72. */
int zenu_hip_init(int device);
/* Release every cached block and the library state. */
int zenu_hip_shutdown(void);
const char *zenu_hip_status_string(int status);
/* hipError_t of the last failed runtime call on this thread, and its text. */
/* The host math library whose results the device's exp, log, tanh, sigmoid, powf, sinh, cosh, sin and
 * cos (f32 and f64) and its f32 tan, asin, acos and atan reproduce bit for bit (the routines are
 * restated from it and compared with it on every f32 argument and on 10^8 to 10^10 sampled f64 ones).  ZeNu's CPU device calls whatever libm the host has: on a host
 * whose libm rounds some of these functions differently (glibc 2.41 and later return correctly
 * rounded results from several f32 functions), CPU and device results differ by the difference between
 * the two libms -- at most 1 ulp for the functions themselves, more for the sigmoid, whose last
 * addition cancels.  No counterpart in the reference. */
const char *zenu_hip_validated_libm(void);
int zenu_hip_last_hip_error(void);
const char *zenu_hip_last_hip_error_string(void);

int zenu_hip_stream_create(zenu_stream_t *stream);   /* runtime/mod.rs:113-121; default priority */
int zenu_hip_stream_destroy(zenu_stream_t stream);
int zenu_hip_stream_synchronize(zenu_stream_t stream);
int zenu_hip_device_synchronize(void);

/* Stream-ordered caching allocator: replaces zenu-matrix/src/memory_pool/mod.rs:79-145 and
 * cuda_malloc_bytes / cuda_free (runtime/mod.rs:30-60, which synchronise the stream on every
 * call).  zenu_hip_malloc never synchronises on a cache hit.  A block freed on stream S is
 * reusable at once by allocations on S; another stream takes it only behind an event (recorded
 * on S at the moment of reuse, waited for by the new stream), never behind a host wait.  `stream`
 * of zenu_hip_free is the last stream that used the block.
 * On out-of-memory the cache is trimmed and the request retried once
 * (the flow zenu-matrix/src/memory_pool/mod.rs:9-20 documents).  Thread-safe.
 * Honours ZENU_USE_MEMPOOL=0 (zenu-matrix/src/lib.rs:36): every call goes to hipMalloc/hipFree;
 * in that mode both functions, and with them every entry point that needs scratch memory, return
 * ZENU_ERR_UNSUPPORTED while `stream` records a graph (hipFree synchronises, and memory freed
 * during a capture would still be written by every replay): nothing is recorded. */
int zenu_hip_malloc(void **ptr_dev, size_t bytes, zenu_stream_t stream);
int zenu_hip_free(void *ptr_dev, zenu_stream_t stream);
/* Stream capture (HIP graphs).  Kernels recorded into a graph keep the addresses they were
 * recorded with and use them again on every replay.  Every block that zenu_hip_malloc hands out
 * while `stream` is capturing -- the library's own scratch (reduction partials, staging copies,
 * the temporaries of zenu_hip_sum_to) as well as the caller's tensors -- is therefore kept out of
 * ordinary requests when it is freed, during the capture or later: only later captures on the
 * same stream may reuse it (graphs recorded on one stream share scratch and must not be
 * replayed concurrently with each other).  After destroying the graphs, call
 * zenu_hip_release_captured(stream) to return those blocks to the pool; zenu_hip_stream_destroy
 * does the same.  A request the pool cannot serve from its cache during a capture goes to
 * hipMalloc, which only the relaxed capture mode tolerates: run the sequence once eagerly on the
 * stream first.  A split reduction on a stream that the library did not create needs its counter
 * ring before the capture starts (any eager reduction on that stream creates it); while
 * capturing, such a call returns ZENU_ERR_UNSUPPORTED instead of blocking.  A captured graph
 * owns a fixed range of its capture stream's counter ring: replay it on that stream, or at
 * least never concurrently with reductions running on that stream.
 * No counterpart in the reference (it never captures). */
int zenu_hip_release_captured(zenu_stream_t stream);
/* Return all cached (free) blocks to the driver. */
int zenu_hip_mempool_trim(void);
typedef struct zenu_mempool_stats {
    uint64_t bytes_in_use;      /* handed out and not yet freed              */
    uint64_t bytes_cached;      /* free blocks held by the pool              */
    uint64_t bytes_reserved;    /* total obtained from the driver            */
    uint64_t n_alloc_calls;     /* zenu_hip_malloc calls                     */
    uint64_t n_cache_hits;      /* of which served from the cache            */
    uint64_t n_driver_allocs;   /* hipMalloc calls                           */
    uint64_t n_driver_frees;    /* hipFree calls                             */
    uint64_t n_oom_retries;     /* allocation retried after a trim           */
} zenu_mempool_stats_t;
int zenu_hip_mempool_stats(zenu_mempool_stats_t *out);

/* Raw driver allocation, bypassing the pool (DeviceBase::raw_alloc / raw_drop_ptr,
 * zenu-matrix/src/device/nvidia/mod.rs:8-16). */
int zenu_hip_raw_malloc(void **ptr_dev, size_t bytes);
int zenu_hip_raw_free(void *ptr_dev);

/* Copies (runtime/mod.rs:83-97).  h2d / d2h return after the host buffer may be reused / read. */
int zenu_hip_memcpy_h2d(void *dst_dev, const void *src_host, size_t bytes, zenu_stream_t stream);
int zenu_hip_memcpy_d2h(void *dst_host, const void *src_dev, size_t bytes, zenu_stream_t stream);
int zenu_hip_memcpy_d2d(void *dst_dev, const void *src_dev, size_t bytes, zenu_stream_t stream);
/* Matrix::zeros: a fill kernel, not BLAS scal-by-0 on uninitialised memory
 * (zenu-matrix/src/device/nvidia/mod.rs:53-58). */
int zenu_hip_memset_zero(void *dst_dev, size_t bytes, zenu_stream_t stream);

/* ------------------------------------------------------------------------- */
/* N-d elementwise ops: one launch per Matrix-level call                       */
/* ------------------------------------------------------------------------- */

/* to = lhs op rhs with ZeNu's broadcasting (add_array / sub_array / mul_array / div_array,
 * zenu-matrix/src/operation/basic_operations.rs:336-374; legality:
 * zenu-matrix/src/with_clousers.rs:155-178, zenu-matrix/src/dim/dim_dyn.rs:24-58,119-148).
 * `to` must have the larger operand's shape. */
int zenu_hip_binary(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *lhs,
                    const zenu_tensor_t *rhs, zenu_stream_t stream);
/* to op= rhs (add_assign ..., basic_operations.rs:318-334; with_clousers.rs:87-153). */
int zenu_hip_binary_assign(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *rhs,
                           zenu_stream_t stream);
/* to = other op scalar (add_scalar ..., basic_operations.rs:291-309); scalar is converted to dtype. */
int zenu_hip_binary_scalar(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                           double scalar, zenu_stream_t stream);
/* to op= scalar (add_scalar_assign ..., basic_operations.rs:310-316). */
int zenu_hip_binary_scalar_assign(int op, int dtype, const zenu_tensor_t *to, double scalar,
                                  zenu_stream_t stream);
/* Same with the scalar read from device memory (the 0-d tensor operand; trait methods
 * scalar_ptr / scalar_assign_ptr, basic_operations.rs:74-88).  No host synchronisation. */
int zenu_hip_binary_scalar_ptr(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                               const void *scalar_dev, zenu_stream_t stream);
int zenu_hip_binary_scalar_assign_ptr(int op, int dtype, const zenu_tensor_t *to,
                                      const void *scalar_dev, zenu_stream_t stream);

/* to = f(other), same shapes (exp_array / log_array / tanh_array / sqrt_array / abs_array ...,
 * basic_operations.rs:512-575); ZENU_SIGMOID is the fused composite. */
int zenu_hip_unary(int fn, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                   zenu_stream_t stream);
int zenu_hip_unary_assign(int fn, int dtype, const zenu_tensor_t *to, zenu_stream_t stream);
/* to = powf(other, scalar) (basic_operations.rs:577-611). */
int zenu_hip_powf(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other, double scalar,
                  zenu_stream_t stream);

/* to = other > 0 ? other : alpha*other ; mask = other > 0 ? 1 : alpha*(-1)
 * (zenu-matrix/src/operation/relu.rs:169-242). */
int zenu_hip_relu(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other, double alpha,
                  zenu_stream_t stream);
int zenu_hip_relu_backward_mask(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                                double alpha, zenu_stream_t stream);

/* gx = gy * mask(x): the two backward ops of zenu-autograd/src/activation/relu.rs:35-44 in one pass. */
int zenu_hip_relu_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gy,
                           const zenu_tensor_t *x, double alpha, zenu_stream_t stream);

/* Backward of tanh and of the sigmoid composite in one pass, with the roundings of the op chains
 * they replace: gx = gy / (cosh(x) * cosh(x)) (zenu-autograd/src/functions/tanh.rs:30-37) and
 * gx = ((0.5 * gy) / (cosh(0.5 * x) * cosh(0.5 * x))) * 0.5 (activation/sigmoid.rs:7-15 through the
 * backward of its mul, tanh, mul and add nodes, functions/mul.rs:35-44).  x is the forward INPUT. */
int zenu_hip_tanh_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gy,
                           const zenu_tensor_t *x, zenu_stream_t stream);
int zenu_hip_sigmoid_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gy,
                              const zenu_tensor_t *x, zenu_stream_t stream);

/* to = clip(other, min, max); mask = 1 inside [min, max] (and for NaN), 0 outside
 * (zenu-matrix/src/operation/clip.rs:289-318).  The assign forms are to == other.  The mask is
 * written with the mask's own stride (clip.rs:90-96 indexes it with the input's). */
int zenu_hip_clip(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other, double min,
                  double max, zenu_stream_t stream);
int zenu_hip_clip_backward_mask(int dtype, const zenu_tensor_t *mask, const zenu_tensor_t *other,
                                double min, double max, zenu_stream_t stream);

/* Strided copy, same shapes (copy_from, zenu-matrix/src/operation/copy_from.rs:211-267;
 * to_default_stride, to_default_stride.rs:7-15). */
int zenu_hip_copy(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *src, zenu_stream_t stream);

/* to = source repeated over to's leading dims and over source dims of size 1 (broadcast,
 * zenu-matrix/src/operation/broadcast.rs:11-43): one launch instead of one copy per slice. */
int zenu_hip_broadcast(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *source,
                       zenu_stream_t stream);

/* ------------------------------------------------------------------------- */
/* Reductions (deterministic: fixed tree, no atomics on data)                  */
/* ------------------------------------------------------------------------- */

/* out = src.sum(axis): out has src's shape without `axis`, or with it kept as size 1
 * (zenu-matrix/src/operation/sum.rs:9-32).  out may be strided. */
int zenu_hip_sum_axis(int dtype, const zenu_tensor_t *out, const zenu_tensor_t *src, int axis,
                      zenu_stream_t stream);
/* zenu_hip_sum_axis for callers that cannot allocate (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same result as
 * zenu_hip_sum_axis, bit for bit (same kernels, same launch geometry), but the call allocates
 * nothing, neither from the driver nor from the caching pool: the arrival counters and partial
 * results of a split reduction and the contiguous staging of a strided destination live in a
 * static device array of 1 040 KiB (16 KiB of counters, 512 KiB of partials, 512 KiB of staging)
 * that the device holds until the process ends.  Limits:
 *   - zenu_hip_init must have run (ZENU_ERR_NOT_INIT otherwise: initialising allocates);
 *   - a source view that zenu_hip_sum_axis would first copy to a contiguous buffer (kept dims
 *     that are neither one uniform stride chain nor a unit-stride run) is refused with
 *     ZENU_ERR_UNSUPPORTED;
 *   - outputs x splits x element size > 512 KiB, more than 4096 counters, or a strided
 *     destination of more than 512 KiB are refused with ZENU_ERR_SCRATCH_LIMIT (a contiguous
 *     destination has no size limit; with 256 compute units no split reduction exceeds 512 KiB
 *     of partials).
 * Every call on the device shares the one array: calls that overlap in time (different streams,
 * or graph replays running concurrently) race and give wrong results; calls ordered on one stream
 * are safe. */
int zenu_hip_sum_axis_noalloc(int dtype, const zenu_tensor_t *out, const zenu_tensor_t *src, int axis,
                              zenu_stream_t stream);
/* Split reductions hand their partial results from many workgroups to one.  That workgroup polls
 * for them; after `polls` fruitless polls (about a microsecond each; default 2^13, about the time
 * one workgroup needs to recompute every split of a 128 MiB reduction) it computes the
 * missing ones itself, so no launch ever depends on the order in which workgroups are dispatched.
 * 0 makes the folding workgroup of every split reduction compute every partial itself without
 * polling at all: a switch for tests, results are the same bits either way.  No counterpart in
 * the reference. */
int zenu_hip_set_reduce_spin_limit(int polls);
/* *count = how many times, since zenu_hip_init, a folding workgroup gave up polling and computed
 * missing partials itself (once per batch of up to 512 partials).  Such launches are correct but
 * can be a poll limit slower than normal; a non-zero count on a GPU that is not shared says that
 * workgroups are being dispatched far out of order.  Blocking (a device-to-host copy).  No
 * counterpart in the reference. */
int zenu_hip_reduce_fallback_count(uint64_t *count);
/* *out_dev = sum of every element (sum_to(x, []), sum.rs:35-94). */
int zenu_hip_sum_all(int dtype, void *out_dev, const zenu_tensor_t *src, zenu_stream_t stream);
/* target = sum_to(src) for any legal target shape (sum.rs:35-94). */
int zenu_hip_sum_to(int dtype, const zenu_tensor_t *target, const zenu_tensor_t *src,
                    zenu_stream_t stream);
/* out = src.max_axis(axis) (zenu-matrix/src/operation/max.rs:67-99). */
int zenu_hip_max_axis(int dtype, const zenu_tensor_t *out, const zenu_tensor_t *src, int axis,
                      zenu_stream_t stream);
/* out_idx_dev[j] = position along `axis` of the FIRST maximum, row-major over the remaining dims
 * (max_axis_idx_ravel, max.rs:103-134); int64 on the ABI, usize in ZeNu. */
int zenu_hip_max_axis_idx(int dtype, int64_t *out_idx_dev, const zenu_tensor_t *src, int axis,
                          zenu_stream_t stream);
/* *out_flat_idx_dev = row-major flat index of the first maximum of the whole view; if
 * out_val_dev is not NULL the maximum itself is stored there (Matrix::max_idx / max_item,
 * max.rs:45-62).  Stays on the device: no host synchronisation. */
int zenu_hip_max_idx(int dtype, int64_t *out_flat_idx_dev, void *out_val_dev,
                     const zenu_tensor_t *src, zenu_stream_t stream);
/* *out_dev = sum |x| (Asum, zenu-matrix/src/operation/asum.rs:14-68). */
int zenu_hip_asum(int dtype, void *out_dev, const zenu_tensor_t *src, zenu_stream_t stream);

/* ------------------------------------------------------------------------- */
/* Fused classifier-head chains (each replaces a sequence of the ops above)    */
/* ------------------------------------------------------------------------- */

/* to = softmax(src) along `axis` (softmax_assign, zenu-matrix/src/operation/softmax.rs:10-25:
 * src - max_axis(axis), exp, / sum(axis)); to may be src. */
int zenu_hip_softmax(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *src, int axis,
                     zenu_stream_t stream);
/* gx = y*gy - y * sum(y*gy, axis) (SoftMax::backward, zenu-autograd/src/loss/softmax.rs:33-40). */
int zenu_hip_softmax_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *y,
                              const zenu_tensor_t *gy, int axis, zenu_stream_t stream);
/* cross_entropy(pred, ans), zenu-autograd/src/loss/cross_entropy.rs:12-23, pred and ans [N, C]:
 * prob = softmax(pred, 1) (kept for the backward pass), loss (0-d) = sum(ans * log(prob)) / -N. */
int zenu_hip_softmax_cross_entropy(int dtype, const zenu_tensor_t *loss, const zenu_tensor_t *prob,
                                   const zenu_tensor_t *pred, const zenu_tensor_t *ans,
                                   zenu_stream_t stream);
/* Gradient of that loss with respect to pred, following the backward of div, sum_to, mul, log
 * and softmax op by op; gloss (0-d, device) is the gradient arriving at the loss, NULL = 1. */
int zenu_hip_softmax_cross_entropy_backward(int dtype, const zenu_tensor_t *gpred,
                                            const zenu_tensor_t *prob, const zenu_tensor_t *ans,
                                            const zenu_tensor_t *gloss, zenu_stream_t stream);
/* pre = z + bias (bias [F] broadcast over the leading dims of z [.., F]), act = relu(pre, alpha):
 * Linear::call followed by relu (zenu-layer/src/layers/linear.rs:27-31,
 * zenu-autograd/src/activation/relu.rs:24-33).  pre may be NULL. */
int zenu_hip_bias_add_relu(int dtype, const zenu_tensor_t *pre, const zenu_tensor_t *act,
                           const zenu_tensor_t *z, const zenu_tensor_t *bias, double alpha,
                           zenu_stream_t stream);
/* The backward pass of a Linear layer needs the gradient of its output and that gradient's column
 * sums (the bias gradient: zenu-layer/src/layers/linear.rs:27-31 through the `sum_to` of
 * zenu-autograd/src/lib.rs:466-486).  Both in one pass over the incoming gradient:
 *   gx = gy * relu'(x)   (zenu_hip_relu_backward),   gbias[j] = sum over every leading index of gx[.., j]
 * gx, gy, x have the same shape [.., N]; gbias holds N elements ([N], [1, N], ..).  One launch (the
 * column-reduction kernel with the ReLU gradient applied to its loads) when the tensors are whole,
 * 16-byte aligned and N is a multiple of the vector width and at least 16; otherwise the two calls it
 * stands for.  gx is bit-identical to zenu_hip_relu_backward's and, for a 2-d gradient, gbias to
 * zenu_hip_sum_to(gbias, gx).
 * No counterpart in the reference (two autograd nodes there). */
int zenu_hip_relu_backward_bias_grad(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gbias,
                                     const zenu_tensor_t *gy, const zenu_tensor_t *x, double alpha,
                                     zenu_stream_t stream);
/* zenu_hip_softmax_cross_entropy_backward that also writes the column sums of gpred to gbias (the bias
 * gradient of the layer that produced the logits).  One launch for a classifier head (at most 256
 * rows, at most 16 classes; each column folded over the rows in a fixed order), otherwise the two
 * calls it stands for.  No counterpart in the reference. */
int zenu_hip_softmax_cross_entropy_backward_bias_grad(int dtype, const zenu_tensor_t *gpred,
                                                      const zenu_tensor_t *gbias, const zenu_tensor_t *prob,
                                                      const zenu_tensor_t *ans, const zenu_tensor_t *gloss,
                                                      zenu_stream_t stream);

/* ------------------------------------------------------------------------- */
/* Fused optimizer updates (one launch, 4 loads + 3 stores per element)        */
/* ------------------------------------------------------------------------- */

/* p -= g*lr (zenu-optimizer/src/sgd.rs:20-31). */
int zenu_hip_sgd_step(int dtype, void *p_dev, const void *g_dev, int64_t n, double lr,
                      zenu_stream_t stream);

/* The same update for n_tensors tensors in one launch (the loop of SGD::update, sgd.rs:20-31):
 * p_dev[i], g_dev[i] are device pointers of sizes[i] elements; host arrays, read during the call. */
int zenu_hip_sgd_step_multi(int dtype, int n_tensors, void *const *p_dev, const void *const *g_dev,
                            const int64_t *sizes, double lr, zenu_stream_t stream);
/* Adam (zenu-optimizer/src/adam.rs:19-59).  `step` is the counter AFTER the increment;
 * 1-beta, beta^step and 1-beta^step are formed on the host in dtype, as the reference does. */
int zenu_hip_adam_step(int dtype, void *p_dev, const void *g_dev, void *m_dev, void *v_dev,
                       int64_t n, double lr, double beta1, double beta2, double eps, double step,
                       zenu_stream_t stream);
/* AdamW (zenu-optimizer/src/adamw.rs:20-70): apply_decay != 0 for keys in weights() only. */
int zenu_hip_adamw_step(int dtype, void *p_dev, const void *g_dev, void *m_dev, void *v_dev,
                        int64_t n, double lr, double beta1, double beta2, double eps,
                        double weight_decay, int apply_decay, double step, zenu_stream_t stream);
/* Multi-tensor form: one launch over a model's parameter tensors.  The pointer / size tables are
 * HOST arrays of length n_tensors; apply_decay may be NULL (no decay) or per-tensor flags.
 * The tables are copied into the kernel arguments (24 tensors per launch): no staging, no
 * synchronisation. */
int zenu_hip_adam_step_multi(int dtype, int n_tensors, void *const *p_dev, const void *const *g_dev,
                             void *const *m_dev, void *const *v_dev, const int64_t *sizes, double lr,
                             double beta1, double beta2, double eps, double weight_decay,
                             const int32_t *apply_decay, double step, zenu_stream_t stream);
/* The same update for callers that record it into a HIP graph.  `Adam::update` advances its step
 * on every call (adam.rs:21-25) and forms 1-beta^step on the host; a recorded launch would replay
 * one step's scalars for ever.  A schedule holds those scalars for steps first_step ..
 * first_step + n_steps - 1 in device memory -- computed on the host in dtype with libm's powf /
 * pow, exactly as the eager call computes them -- and a cursor, also in device memory, that every
 * scheduled update advances (a one-thread launch after the update's own).  A recorded scheduled
 * update is therefore the NEXT step on every replay, bit for bit what consecutive eager calls
 * give.  An update asked for after the last step of the table changes nothing and is counted
 * (`refused` of the query): create a new schedule from `next_step` before that happens.
 * create / destroy / query block and may not be called while `stream` records a graph; the
 * scheduled update never blocks and allocates nothing.  One device array per schedule
 * (16 bytes + 2 elements per step).  No counterpart in the reference. */
int zenu_hip_adam_schedule_create(void **schedule, int dtype, double beta1, double beta2,
                                  int64_t first_step, int n_steps, zenu_stream_t stream);
int zenu_hip_adam_schedule_destroy(void *schedule, zenu_stream_t stream);
/* any of the three outputs may be NULL */
int zenu_hip_adam_schedule_query(void *schedule, int64_t *next_step, int64_t *steps_left,
                                 int64_t *refused, zenu_stream_t stream);
/* zenu_hip_adam_step_multi with beta1, beta2 and the step taken from `schedule` */
int zenu_hip_adam_step_multi_scheduled(int dtype, int n_tensors, void *const *p_dev,
                                       const void *const *g_dev, void *const *m_dev,
                                       void *const *v_dev, const int64_t *sizes, double lr, double eps,
                                       double weight_decay, const int32_t *apply_decay, void *schedule,
                                       zenu_stream_t stream);

/* ------------------------------------------------------------------------- */
/* Entry points with the reference's own names and argument order              */
/* (the headers under zenu-cuda-kernel-sys/kernel/): 1-D, int sizes/strides, null stream. */
/* They let the unchanged zenu-cuda/src/kernel/mod.rs wrappers link.            */
/* ------------------------------------------------------------------------- */

/* The reference's functions return void (the headers under kernel/) and so do these; what the descriptor entry
 * point behind one of them returned is kept per thread instead.  zenu_hip_last_status() returns
 * the first status other than ZENU_OK that any of them produced on this thread since the last
 * call, and clears it: a wrapper can poll it after a batch of calls (no counterpart in the
 * reference, whose kernels check nothing). */
/* Self-check of the device math: f32 tanh, sigmoid, sinh, cosh, tan, atan, asin and acos (fn = the
 * zenu_unop_t value) use a 4-instruction division / square root that is exact only on the operands
 * these functions produce.  The call evaluates the function on ALL 2^32 f32 bit patterns twice on
 * the device -- as shipped, and with the IEEE division and square root in the same places -- and
 * returns in *mismatches how many results differ (0 is the only acceptable answer) and in
 * *example_bits (may be NULL) the bit pattern of one argument that differs.  fn = 1000 / 1001
 * compare the bare division / square root on operands of every exponent, where they do differ
 * (the short forms have no operand scaling): a check of the check.  Blocking; a few tens of milliseconds per function.  No counterpart in the reference. */
int zenu_hip_selfcheck_short_division(int fn, uint64_t *mismatches, uint32_t *example_bits,
                                      zenu_stream_t stream);
/* Every f32 bit pattern of [first, first + count) through unary function fn (a zenu_unop_t value:
 * exp, log, tanh, sigmoid, sin, cos, tan, asin, acos, atan, sinh, cosh -- the functions whose results are
 * meant to be a host libm's bits), folded on the device into one 64-bit sum per block of
 * 2^block_log2 patterns (8 <= block_log2 <= 32; count a multiple of the block size):
 * sums_dev[b] = sum over the block of T(argument bits, result bits) mod 2^64, T = the finalizer of
 * splitmix64 applied to (argument << 32 | result), every NaN result counted as 0x7fc00000.  A
 * caller that folds the results of ITS libm the same way learns, without copying a result, whether
 * the device returns that libm's bits on every argument (the whole range takes the device 0.1-0.2 s
 * per function; 16 host threads need 10-20 s).  Asynchronous on `stream`.  No counterpart in the
 * reference. */
int zenu_hip_unary_range_hash(int fn, uint64_t first, uint64_t count, int block_log2,
                              uint64_t *sums_dev, zenu_stream_t stream);
/* The same for powf(x, exponent) over the f32 bases x. */
int zenu_hip_powf_range_hash(double exponent, uint64_t first, uint64_t count, int block_log2,
                             uint64_t *sums_dev, zenu_stream_t stream);
/* The same for the f64 functions whose results are meant to be a host libm's bits (exp, log, tanh,
 * sigmoid, sinh, cosh, sin, cos) on SAMPLED arguments: argument number i of [first, first + count) has the high word
 * (sign, exponent, 20 mantissa bits) (uint32_t)(i * step + offset) and the low word
 * (uint32_t)(((i + salt) * 0x9E3779B97F4A7C15) >> 29); the term is M(M(argument bits) + result bits)
 * with M the finalizer of splitmix64 and every NaN result counted as 0x7ff8000000000000. */
int zenu_hip_unary_range_hash_f64(int fn, uint64_t first, uint64_t count, int block_log2, uint32_t step,
                                  uint32_t offset, uint64_t salt, uint64_t *sums_dev,
                                  zenu_stream_t stream);
/* The same for the f64 powf(x, exponent) over sampled bases x. */
int zenu_hip_powf_range_hash_f64(double exponent, uint64_t first, uint64_t count, int block_log2,
                                 uint32_t step, uint32_t offset, uint64_t salt, uint64_t *sums_dev,
                                 zenu_stream_t stream);
int zenu_hip_last_status(void);

#define ZENU_DECL_1D(T, S)                                                                        \
    /* array_array.h:7-28 */                                                                      \
    void array_array_add_##S(T *a, int stride_a, T *b, int stride_b, T *c, int stride_c, int n);  \
    void array_array_sub_##S(T *a, int stride_a, T *b, int stride_b, T *c, int stride_c, int n);  \
    void array_array_mul_##S(T *a, int stride_a, T *b, int stride_b, T *c, int stride_c, int n);  \
    void array_array_div_##S(T *a, int stride_a, T *b, int stride_b, T *c, int stride_c, int n);  \
    void array_array_add_assign_##S(T *a, int stride_a, T *b, int stride_b, int n);               \
    void array_array_sub_assign_##S(T *a, int stride_a, T *b, int stride_b, int n);               \
    void array_array_mul_assign_##S(T *a, int stride_a, T *b, int stride_b, int n);               \
    void array_array_div_assign_##S(T *a, int stride_a, T *b, int stride_b, int n);               \
    /* array_scalar.h:7-44 */                                                                     \
    void array_scalar_add_##S(T *a, int size, int stride_a, T scalar, T *out, int stride_out);    \
    void array_scalar_sub_##S(T *a, int size, int stride_a, T scalar, T *out, int stride_out);    \
    void array_scalar_mul_##S(T *a, int size, int stride_a, T scalar, T *out, int stride_out);    \
    void array_scalar_div_##S(T *a, int size, int stride_a, T scalar, T *out, int stride_out);    \
    void array_scalar_add_assign_##S(T *a, int size, int stride, T scalar);                       \
    void array_scalar_sub_assign_##S(T *a, int size, int stride, T scalar);                       \
    void array_scalar_mul_assign_##S(T *a, int size, int stride, T scalar);                       \
    void array_scalar_div_assign_##S(T *a, int size, int stride, T scalar);                       \
    void array_scalar_pointer_add_##S(T *a, int size, int stride_a, T *scalar, T *out, int stride_out); \
    void array_scalar_pointer_sub_##S(T *a, int size, int stride_a, T *scalar, T *out, int stride_out); \
    void array_scalar_pointer_mul_##S(T *a, int size, int stride_a, T *scalar, T *out, int stride_out); \
    void array_scalar_pointer_div_##S(T *a, int size, int stride_a, T *scalar, T *out, int stride_out); \
    void array_scalar_pointer_add_assign_##S(T *a, int size, int stride, T *scalar);              \
    void array_scalar_pointer_sub_assign_##S(T *a, int size, int stride, T *scalar);              \
    void array_scalar_pointer_mul_assign_##S(T *a, int size, int stride, T *scalar);              \
    void array_scalar_pointer_div_assign_##S(T *a, int size, int stride, T *scalar);              \
    /* array_scalar.h:46-112 (unary) */                                                           \
    void array_exp_##S(T *a, int size, int stride_in, T *out, int stride_out);                    \
    void array_log_##S(T *a, int size, int stride_in, T *out, int stride_out);                    \
    void array_tanh_##S(T *a, int size, int stride_in, T *out, int stride_out);                   \
    void array_sqrt_##S(T *a, int size, int stride_in, T *out, int stride_out);                   \
    void array_abs_##S(T *a, int size, int stride_in, T *out, int stride_out);                    \
    void array_exp_assign_##S(T *a, int size, int stride);                                        \
    void array_log_assign_##S(T *a, int size, int stride);                                        \
    void array_tanh_assign_##S(T *a, int size, int stride);                                       \
    void array_sqrt_assign_##S(T *a, int size, int stride);                                       \
    void array_abs_assign_##S(T *a, int size, int stride);                                        \
    void array_sin_##S(T *a, int size, int stride_in, T *out, int stride_out);                    \
    void array_cos_##S(T *a, int size, int stride_in, T *out, int stride_out);                    \
    void array_tan_##S(T *a, int size, int stride_in, T *out, int stride_out);                    \
    void array_asin_##S(T *a, int size, int stride_in, T *out, int stride_out);                   \
    void array_acos_##S(T *a, int size, int stride_in, T *out, int stride_out);                   \
    void array_atan_##S(T *a, int size, int stride_in, T *out, int stride_out);                   \
    void array_sinh_##S(T *a, int size, int stride_in, T *out, int stride_out);                   \
    void array_cosh_##S(T *a, int size, int stride_in, T *out, int stride_out);                   \
    void array_sin_assign_##S(T *a, int size, int stride);                                        \
    void array_cos_assign_##S(T *a, int size, int stride);                                        \
    void array_tan_assign_##S(T *a, int size, int stride);                                        \
    void array_asin_assign_##S(T *a, int size, int stride);                                       \
    void array_acos_assign_##S(T *a, int size, int stride);                                       \
    void array_atan_assign_##S(T *a, int size, int stride);                                       \
    void array_sinh_assign_##S(T *a, int size, int stride);                                       \
    void array_cosh_assign_##S(T *a, int size, int stride);                                       \
    /* array_scalar.h:109-112 */                                                                  \
    void array_pow_##S(T *a, int size, int stride_a, T scalar, T *out, int stride_o);             \
    void array_pow_assign_##S(T *a, int size, int stride, T scalar);                              \
    /* array_scalar.h:97-106 */                                                                   \
    void array_clip_##S(T *input, T *output, int size, int stride_in, int stride_out, T min, T max); \
    void array_clip_assign_##S(T *input, int size, int stride, T min, T max);                     \
    void array_clip_backward_##S(T *input, T *mask, T max, T min, int size, int stride_in,        \
                                 int stride_mask);                                                \
    void array_clip_backward_assign_##S(T *input, T max, T min, int size, int stride);            \
    /* array_array.h:27-28: output[i] = input[i] + bias[(i / channel_stride) % bias_size] */      \
    void conv_bias_add_##S(const T *input, T *output, int channel_stride, const T *bias,          \
                           int bias_size, int total_elements);                                    \
    /* conv2d_bkwd_data.h:7-17: dbias[c] = sum over n, h, w of dOut[n, c, h, w]; follows the CPU  \
       path (zenu-matrix/src/nn/conv/cpu/bias.rs:18-25: sum(0), sum(2), sum(3)) */                \
    void conv2d_bias_bkwd_##S(const T *dOut, T *dbias, int N, int C, int H, int W);               \
    /* activations.h:7-11 */                                                                      \
    void relu_##S(T *input, T *output, T alpha, int size, int input_stride, int output_stride);   \
    void relu_backward_mask_##S(T *input, T *mask, T alpha, int size, int input_stride,           \
                                int mask_stride);                                                 \
    /* element_wise.h:7-9: `out` is a HOST int (zenu-cuda/src/kernel/mod.rs:570-588); blocking */ \
    void array_max_idx_##S(T *a, int size, int stride, int *out);                                 \
    /* memory_access.h:7-11: blocking single-element copies */                                    \
    void memory_access_##S(T *array, int offset, T *result);                                      \
    void memory_set_##S(T *array, int offset, T value);

ZENU_DECL_1D(float, float)
ZENU_DECL_1D(double, double)

#ifdef __cplusplus
}
#endif
#endif /* ZENU_HIP_H */
