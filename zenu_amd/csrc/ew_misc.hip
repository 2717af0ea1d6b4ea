// ew_misc.hip -- relu and its masks, the one-pass activation backward passes, clip, broadcast and
// strided copy (zenu-matrix/src/operation/{relu.rs:169-242, clip.rs:289-318, broadcast.rs:11-43,
// copy_from.rs:211-267}); engine in elementwise.hpp.
#include "elementwise.hpp"

using namespace zenu;


template <template <typename> class F>
static int activation_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gy, const zenu_tensor_t *x,
                               zenu_stream_t stream)
{
    int rc = check2(gx, gy);
    if (!rc) rc = validate_tensor(x);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*gx, *gy) || !same_shape(*gx, *x)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) return run2<float>(*gx, *gy, *x, F<float>(), as_stream(stream));
    if (dtype == ZENU_F64) return run2<double>(*gx, *gy, *x, F<double>(), as_stream(stream));
    return ZENU_ERR_ARG;
}

extern "C" {

int zenu_hip_relu(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other, double alpha,
                  zenu_stream_t stream)
{
    int rc = check2(to, other);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*to, *other)) return ZENU_ERR_SHAPE;  // "shape mismatch"
    if (dtype == ZENU_F32) { ReluF<float> f; f.alpha = (float)alpha; return run1<float>(*to, *other, f, as_stream(stream)); }
    if (dtype == ZENU_F64) { ReluF<double> f; f.alpha = alpha; return run1<double>(*to, *other, f, as_stream(stream)); }
    return ZENU_ERR_ARG;
}

int zenu_hip_relu_backward_mask(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                                double alpha, zenu_stream_t stream)
{
    int rc = check2(to, other);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*to, *other)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) { ReluMaskF<float> f; f.alpha = (float)alpha; return run1<float>(*to, *other, f, as_stream(stream)); }
    if (dtype == ZENU_F64) { ReluMaskF<double> f; f.alpha = alpha; return run1<double>(*to, *other, f, as_stream(stream)); }
    return ZENU_ERR_ARG;
}

int zenu_hip_broadcast(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *source, zenu_stream_t stream)
{
    int rc = check2(to, source);
    if (!rc) rc = ensure_init();
    if (!rc) rc = check_broadcast(*to, *source);   // broadcast.rs:11-43: the test at :13-17 and what its recursion then requires
    if (rc) return rc;
    if (dtype == ZENU_F32) return run1<float>(*to, *source, CopyF<float>(), as_stream(stream));
    if (dtype == ZENU_F64) return run1<double>(*to, *source, CopyF<double>(), as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_relu_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gy, const zenu_tensor_t *x,
                           double alpha, zenu_stream_t stream)
{
    int rc = check2(gx, gy);
    if (!rc) rc = validate_tensor(x);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*gx, *gy) || !same_shape(*gx, *x)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) { ReluBwdF<float> f; f.alpha = (float)alpha; return run2<float>(*gx, *gy, *x, f, as_stream(stream)); }
    if (dtype == ZENU_F64) { ReluBwdF<double> f; f.alpha = alpha; return run2<double>(*gx, *gy, *x, f, as_stream(stream)); }
    return ZENU_ERR_ARG;
}

int zenu_hip_tanh_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gy, const zenu_tensor_t *x,
                           zenu_stream_t stream)
{
    return activation_backward<TanhBwdF>(dtype, gx, gy, x, stream);
}

int zenu_hip_sigmoid_backward(int dtype, const zenu_tensor_t *gx, const zenu_tensor_t *gy, const zenu_tensor_t *x,
                              zenu_stream_t stream)
{
    return activation_backward<SigmoidBwdF>(dtype, gx, gy, x, stream);
}

int zenu_hip_clip(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other, double min, double max,
                  zenu_stream_t stream)
{
    int rc = check2(to, other);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*to, *other)) return ZENU_ERR_SHAPE;
    if (to->ndim == 0) return ZENU_ERR_RANK;   // clip.rs:213-214: a 0-d input is unimplemented!() in the reference
    if (dtype == ZENU_F32) { ClipF<float> f; f.lo = (float)min; f.hi = (float)max; return run1<float>(*to, *other, f, as_stream(stream)); }
    if (dtype == ZENU_F64) { ClipF<double> f; f.lo = min; f.hi = max; return run1<double>(*to, *other, f, as_stream(stream)); }
    return ZENU_ERR_ARG;
}

int zenu_hip_clip_backward_mask(int dtype, const zenu_tensor_t *mask, const zenu_tensor_t *other, double min,
                                double max, zenu_stream_t stream)
{
    int rc = check2(mask, other);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*mask, *other)) return ZENU_ERR_SHAPE;
    if (mask->ndim == 0) return ZENU_ERR_RANK;   // clip.rs:251-252, as above
    if (dtype == ZENU_F32) { ClipMaskF<float> f; f.lo = (float)min; f.hi = (float)max; return run1<float>(*mask, *other, f, as_stream(stream)); }
    if (dtype == ZENU_F64) { ClipMaskF<double> f; f.lo = min; f.hi = max; return run1<double>(*mask, *other, f, as_stream(stream)); }
    return ZENU_ERR_ARG;
}

int zenu_hip_copy(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *src, zenu_stream_t stream)
{
    int rc = check2(to, src);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*to, *src)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) return run1<float>(*to, *src, CopyF<float>(), as_stream(stream));
    if (dtype == ZENU_F64) return run1<double>(*to, *src, CopyF<double>(), as_stream(stream));
    return ZENU_ERR_ARG;
}

}  // extern "C"
