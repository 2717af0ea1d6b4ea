// shims.cpp -- the reference's own 1-D entry points (zenu-cuda-kernel-sys/kernel/*.h), so the
// unchanged wrappers of zenu-cuda/src/kernel/mod.rs and kernel/activation.rs link against this
// library.  Same names, same argument order, `int` sizes and element strides, launches on the
// null stream, no return value (the reference's functions return void and check nothing).
// Each one forwards to the N-d entry point with a 1-D strided view.  A status that the void
// signature cannot return is kept per thread: the first failure since the last call of
// zenu_hip_last_status() stays there until that call reads and clears it.
#include "common.hpp"

namespace {

thread_local int tl_sticky_status = ZENU_OK;
inline void note(int rc)
{
    if (rc != ZENU_OK && tl_sticky_status == ZENU_OK) tl_sticky_status = rc;
}

zenu_tensor_t view1d(const void *p, int n, int stride)
{
    zenu_tensor_t t;
    t.ptr = const_cast<void *>(p);
    t.ndim = 1;
    t.reserved = 0;
    for (int i = 0; i < ZENU_MAX_DIM; i++) { t.shape[i] = 0; t.stride[i] = 0; }
    t.shape[0] = n;
    t.stride[0] = stride;
    return t;
}

template <typename T> constexpr int dtype_of();
template <> constexpr int dtype_of<float>() { return ZENU_F32; }
template <> constexpr int dtype_of<double>() { return ZENU_F64; }

template <typename T>
void aa(int op, T *a, int sa, T *b, int sb, T *c, int sc, int n)
{
    zenu_tensor_t ta = view1d(a, n, sa), tb = view1d(b, n, sb), tc = view1d(c, n, sc);
    note(zenu_hip_binary(op, dtype_of<T>(), &tc, &ta, &tb, nullptr));
}
template <typename T> void aa_assign(int op, T *a, int sa, T *b, int sb, int n)
{
    zenu_tensor_t ta = view1d(a, n, sa), tb = view1d(b, n, sb);
    note(zenu_hip_binary_assign(op, dtype_of<T>(), &ta, &tb, nullptr));
}
template <typename T> void as(int op, T *a, int n, int sa, T s, T *out, int so)
{
    zenu_tensor_t ta = view1d(a, n, sa), to = view1d(out, n, so);
    note(zenu_hip_binary_scalar(op, dtype_of<T>(), &to, &ta, (double)s, nullptr));
}
template <typename T> void as_assign(int op, T *a, int n, int sa, T s)
{
    zenu_tensor_t ta = view1d(a, n, sa);
    note(zenu_hip_binary_scalar_assign(op, dtype_of<T>(), &ta, (double)s, nullptr));
}
template <typename T> void asp(int op, T *a, int n, int sa, T *s, T *out, int so)
{
    zenu_tensor_t ta = view1d(a, n, sa), to = view1d(out, n, so);
    note(zenu_hip_binary_scalar_ptr(op, dtype_of<T>(), &to, &ta, s, nullptr));
}
template <typename T> void asp_assign(int op, T *a, int n, int sa, T *s)
{
    zenu_tensor_t ta = view1d(a, n, sa);
    note(zenu_hip_binary_scalar_assign_ptr(op, dtype_of<T>(), &ta, s, nullptr));
}
template <typename T> void un(int fn, T *a, int n, int si, T *out, int so)
{
    zenu_tensor_t ta = view1d(a, n, si), to = view1d(out, n, so);
    note(zenu_hip_unary(fn, dtype_of<T>(), &to, &ta, nullptr));
}
template <typename T> void un_assign(int fn, T *a, int n, int s)
{
    zenu_tensor_t ta = view1d(a, n, s);
    note(zenu_hip_unary_assign(fn, dtype_of<T>(), &ta, nullptr));
}

zenu_tensor_t view3d(const void *p, int64_t d0, int64_t d1, int64_t d2, int64_t s0, int64_t s1, int64_t s2)
{
    zenu_tensor_t t = view1d(p, 0, 0);
    t.ndim = 3;
    t.shape[0] = d0; t.shape[1] = d1; t.shape[2] = d2;
    t.stride[0] = s0; t.stride[1] = s1; t.stride[2] = s2;
    return t;
}

// output[i] = input[i] + bias[(i / channel_stride) % bias_size] (array_array.cu:49-57) as broadcast
// adds: whole [C, channel_stride] images, then the channels and the partial channel left over
template <typename T>
void conv_bias(const T *in, T *out, int cs, const T *bias, int C, int total)
{
    if (cs <= 0 || C <= 0 || total <= 0) return;
    const int64_t image = (int64_t)C * cs;
    const int64_t images = total / image;
    if (images > 0) {
        zenu_tensor_t ti = view3d(in, images, C, cs, image, cs, 1), to = view3d(out, images, C, cs, image, cs, 1);
        zenu_tensor_t tb = view3d(bias, 1, C, 1, C, 1, 1);
        note(zenu_hip_binary(ZENU_ADD, dtype_of<T>(), &to, &ti, &tb, nullptr));
    }
    int64_t done = images * image;
    const int64_t chans = (total - done) / cs;
    if (chans > 0) {
        zenu_tensor_t ti = view3d(in + done, 1, chans, cs, image, cs, 1), to = view3d(out + done, 1, chans, cs, image, cs, 1);
        zenu_tensor_t tb = view3d(bias, 1, chans, 1, C, 1, 1);
        note(zenu_hip_binary(ZENU_ADD, dtype_of<T>(), &to, &ti, &tb, nullptr));
        done += chans * cs;
    }
    if (done < total) {
        zenu_tensor_t ti = view1d(in + done, (int)(total - done), 1), to = view1d(out + done, (int)(total - done), 1);
        note(zenu_hip_binary_scalar_ptr(ZENU_ADD, dtype_of<T>(), &to, &ti, bias + chans, nullptr));
    }
}

// d_bias[c] = sum over n, h, w of d_output[n, c, h, w] (NCHW, contiguous), as the CPU path defines it:
// sum(0), sum(2), sum(3) in that order (zenu-matrix/src/nn/conv/cpu/bias.rs:18-25).  The CUDA kernel
// of the same name (conv2d_bkwd_data.cu:120-156) reads channel c as ONE run of N*H*W elements, which
// is that sum only for N = 1; the CPU path is the one followed.
template <typename T> void conv_bias_bkwd(const T *dout, T *dbias, int N, int C, int H, int W)
{
    if (C <= 0) return;
    zenu_tensor_t src = view1d(dout, 0, 0), dst = view1d(dbias, 0, 0);
    src.ndim = dst.ndim = 4;
    const int64_t shape[4] = {N, C, H, W};
    int64_t st = 1;
    for (int i = 3; i >= 0; i--) {
        src.shape[i] = shape[i];
        src.stride[i] = st;
        st *= shape[i];
        dst.shape[i] = (i == 1) ? C : 1;
        dst.stride[i] = (i == 0) ? C : 1;
    }
    note(zenu_hip_sum_to(dtype_of<T>(), &dst, &src, nullptr));
}

template <typename T> void max_idx(T *a, int size, int stride, int *out)
{
    // `out` is host memory (zenu-cuda/src/kernel/mod.rs:570-588): blocking, like the reference
    zenu_tensor_t ta = view1d(a, size, stride);
    void *d = nullptr;
    int rc = zenu_hip_malloc(&d, sizeof(int64_t), nullptr);
    if (rc != ZENU_OK) { note(rc); return; }
    int64_t h = 0;
    rc = zenu_hip_max_idx(dtype_of<T>(), static_cast<int64_t *>(d), nullptr, &ta, nullptr);
    if (rc == ZENU_OK) rc = zenu_hip_memcpy_d2h(&h, d, sizeof h, nullptr);
    if (rc == ZENU_OK) *out = (int)h;
    note(rc);
    note(zenu_hip_free(d, nullptr));
}

}  // namespace

extern "C" {

int zenu_hip_last_status(void)
{
    const int rc = tl_sticky_status;
    tl_sticky_status = ZENU_OK;
    return rc;
}

#define ZENU_DEF_1D(T, S)                                                                                  \
    void array_array_add_##S(T *a, int sa, T *b, int sb, T *c, int sc, int n) { aa<T>(ZENU_ADD, a, sa, b, sb, c, sc, n); } \
    void array_array_sub_##S(T *a, int sa, T *b, int sb, T *c, int sc, int n) { aa<T>(ZENU_SUB, a, sa, b, sb, c, sc, n); } \
    void array_array_mul_##S(T *a, int sa, T *b, int sb, T *c, int sc, int n) { aa<T>(ZENU_MUL, a, sa, b, sb, c, sc, n); } \
    void array_array_div_##S(T *a, int sa, T *b, int sb, T *c, int sc, int n) { aa<T>(ZENU_DIV, a, sa, b, sb, c, sc, n); } \
    void array_array_add_assign_##S(T *a, int sa, T *b, int sb, int n) { aa_assign<T>(ZENU_ADD, a, sa, b, sb, n); } \
    void array_array_sub_assign_##S(T *a, int sa, T *b, int sb, int n) { aa_assign<T>(ZENU_SUB, a, sa, b, sb, n); } \
    void array_array_mul_assign_##S(T *a, int sa, T *b, int sb, int n) { aa_assign<T>(ZENU_MUL, a, sa, b, sb, n); } \
    void array_array_div_assign_##S(T *a, int sa, T *b, int sb, int n) { aa_assign<T>(ZENU_DIV, a, sa, b, sb, n); } \
    void array_scalar_add_##S(T *a, int n, int sa, T s, T *o, int so) { as<T>(ZENU_ADD, a, n, sa, s, o, so); } \
    void array_scalar_sub_##S(T *a, int n, int sa, T s, T *o, int so) { as<T>(ZENU_SUB, a, n, sa, s, o, so); } \
    void array_scalar_mul_##S(T *a, int n, int sa, T s, T *o, int so) { as<T>(ZENU_MUL, a, n, sa, s, o, so); } \
    void array_scalar_div_##S(T *a, int n, int sa, T s, T *o, int so) { as<T>(ZENU_DIV, a, n, sa, s, o, so); } \
    void array_scalar_add_assign_##S(T *a, int n, int sa, T s) { as_assign<T>(ZENU_ADD, a, n, sa, s); } \
    void array_scalar_sub_assign_##S(T *a, int n, int sa, T s) { as_assign<T>(ZENU_SUB, a, n, sa, s); } \
    void array_scalar_mul_assign_##S(T *a, int n, int sa, T s) { as_assign<T>(ZENU_MUL, a, n, sa, s); } \
    void array_scalar_div_assign_##S(T *a, int n, int sa, T s) { as_assign<T>(ZENU_DIV, a, n, sa, s); } \
    void array_scalar_pointer_add_##S(T *a, int n, int sa, T *s, T *o, int so) { asp<T>(ZENU_ADD, a, n, sa, s, o, so); } \
    void array_scalar_pointer_sub_##S(T *a, int n, int sa, T *s, T *o, int so) { asp<T>(ZENU_SUB, a, n, sa, s, o, so); } \
    void array_scalar_pointer_mul_##S(T *a, int n, int sa, T *s, T *o, int so) { asp<T>(ZENU_MUL, a, n, sa, s, o, so); } \
    void array_scalar_pointer_div_##S(T *a, int n, int sa, T *s, T *o, int so) { asp<T>(ZENU_DIV, a, n, sa, s, o, so); } \
    void array_scalar_pointer_add_assign_##S(T *a, int n, int sa, T *s) { asp_assign<T>(ZENU_ADD, a, n, sa, s); } \
    void array_scalar_pointer_sub_assign_##S(T *a, int n, int sa, T *s) { asp_assign<T>(ZENU_SUB, a, n, sa, s); } \
    void array_scalar_pointer_mul_assign_##S(T *a, int n, int sa, T *s) { asp_assign<T>(ZENU_MUL, a, n, sa, s); } \
    void array_scalar_pointer_div_assign_##S(T *a, int n, int sa, T *s) { asp_assign<T>(ZENU_DIV, a, n, sa, s); } \
    void array_exp_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_EXP, a, n, si, o, so); }            \
    void array_log_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_LOG, a, n, si, o, so); }            \
    void array_tanh_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_TANH, a, n, si, o, so); }          \
    void array_sqrt_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_SQRT, a, n, si, o, so); }          \
    void array_abs_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_ABS, a, n, si, o, so); }            \
    void array_exp_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_EXP, a, n, s); }                     \
    void array_log_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_LOG, a, n, s); }                     \
    void array_tanh_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_TANH, a, n, s); }                   \
    void array_sqrt_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_SQRT, a, n, s); }                   \
    void array_abs_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_ABS, a, n, s); }                     \
    void array_sin_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_SIN, a, n, si, o, so); }            \
    void array_cos_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_COS, a, n, si, o, so); }            \
    void array_tan_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_TAN, a, n, si, o, so); }            \
    void array_asin_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_ASIN, a, n, si, o, so); }          \
    void array_acos_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_ACOS, a, n, si, o, so); }          \
    void array_atan_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_ATAN, a, n, si, o, so); }          \
    void array_sinh_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_SINH, a, n, si, o, so); }          \
    void array_cosh_##S(T *a, int n, int si, T *o, int so) { un<T>(ZENU_COSH, a, n, si, o, so); }          \
    void array_sin_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_SIN, a, n, s); }                     \
    void array_cos_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_COS, a, n, s); }                     \
    void array_tan_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_TAN, a, n, s); }                     \
    void array_asin_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_ASIN, a, n, s); }                   \
    void array_acos_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_ACOS, a, n, s); }                   \
    void array_atan_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_ATAN, a, n, s); }                   \
    void array_sinh_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_SINH, a, n, s); }                   \
    void array_cosh_assign_##S(T *a, int n, int s) { un_assign<T>(ZENU_COSH, a, n, s); }                   \
    void array_pow_##S(T *a, int n, int sa, T scalar, T *o, int so)                                        \
    {                                                                                                      \
        zenu_tensor_t ti = view1d(a, n, sa), to = view1d(o, n, so);                                        \
        note(zenu_hip_powf(dtype_of<T>(), &to, &ti, (double)scalar, nullptr));                             \
    }                                                                                                      \
    void array_pow_assign_##S(T *a, int n, int s, T scalar)                                                \
    {                                                                                                      \
        zenu_tensor_t t = view1d(a, n, s);                                                                 \
        note(zenu_hip_powf(dtype_of<T>(), &t, &t, (double)scalar, nullptr));                               \
    }                                                                                                      \
    void array_clip_##S(T *in, T *out, int n, int si, int so, T lo, T hi)                                  \
    {                                                                                                      \
        zenu_tensor_t ti = view1d(in, n, si), to = view1d(out, n, so);                                     \
        note(zenu_hip_clip(dtype_of<T>(), &to, &ti, (double)lo, (double)hi, nullptr));                     \
    }                                                                                                      \
    void array_clip_assign_##S(T *a, int n, int s, T lo, T hi)                                             \
    {                                                                                                      \
        zenu_tensor_t t = view1d(a, n, s);                                                                 \
        note(zenu_hip_clip(dtype_of<T>(), &t, &t, (double)lo, (double)hi, nullptr));                       \
    }                                                                                                      \
    void array_clip_backward_##S(T *in, T *mask, T hi, T lo, int n, int si, int sm)                        \
    {                                                                                                      \
        zenu_tensor_t ti = view1d(in, n, si), tm = view1d(mask, n, sm);                                    \
        note(zenu_hip_clip_backward_mask(dtype_of<T>(), &tm, &ti, (double)lo, (double)hi, nullptr));       \
    }                                                                                                      \
    void array_clip_backward_assign_##S(T *a, T hi, T lo, int n, int s)                                    \
    {                                                                                                      \
        zenu_tensor_t t = view1d(a, n, s);                                                                 \
        note(zenu_hip_clip_backward_mask(dtype_of<T>(), &t, &t, (double)lo, (double)hi, nullptr));         \
    }                                                                                                      \
    void conv_bias_add_##S(const T *in, T *out, int channel_stride, const T *bias, int bias_size, int total) \
    {                                                                                                      \
        conv_bias<T>(in, out, channel_stride, bias, bias_size, total);                                     \
    }                                                                                                      \
    void conv2d_bias_bkwd_##S(const T *dout, T *dbias, int N, int C, int H, int W)                         \
    {                                                                                                      \
        conv_bias_bkwd<T>(dout, dbias, N, C, H, W);                                                        \
    }                                                                                                      \
    void relu_##S(T *in, T *out, T alpha, int n, int si, int so)                                           \
    {                                                                                                      \
        zenu_tensor_t ti = view1d(in, n, si), to = view1d(out, n, so);                                     \
        note(zenu_hip_relu(dtype_of<T>(), &to, &ti, (double)alpha, nullptr));                              \
    }                                                                                                      \
    void relu_backward_mask_##S(T *in, T *mask, T alpha, int n, int si, int sm)                            \
    {                                                                                                      \
        zenu_tensor_t ti = view1d(in, n, si), tm = view1d(mask, n, sm);                                    \
        note(zenu_hip_relu_backward_mask(dtype_of<T>(), &tm, &ti, (double)alpha, nullptr));                \
    }                                                                                                      \
    void array_max_idx_##S(T *a, int size, int stride, int *out) { max_idx<T>(a, size, stride, out); }     \
    void memory_access_##S(T *array, int offset, T *result)                                                \
    {                                                                                                      \
        note(zenu_hip_memcpy_d2h(result, array + offset, sizeof(T), nullptr));                             \
    }                                                                                                      \
    void memory_set_##S(T *array, int offset, T value)                                                     \
    {                                                                                                      \
        note(zenu_hip_memcpy_h2d(array + offset, &value, sizeof(T), nullptr));                             \
    }

ZENU_DEF_1D(float, float)
ZENU_DEF_1D(double, double)

}  // extern "C"
