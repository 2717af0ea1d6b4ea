// ew_unary.hip -- entry points of the unary operators and powf
// (zenu-matrix/src/operation/basic_operations.rs:383-611); engine in elementwise.hpp.  The
// trigonometric and hyperbolic functions are instantiated in ew_unary_trig.hip.
#include "elementwise.hpp"

namespace zenu {

int unary_trig(int dtype, int fn, const zenu_tensor_t &to, const zenu_tensor_t &in, hipStream_t s);

namespace {

template <typename T> struct ZenuDType;
template <> struct ZenuDType<float> { static constexpr int value = ZENU_F32; };
template <> struct ZenuDType<double> { static constexpr int value = ZENU_F64; };

template <typename T> int unary_t(int fn, const zenu_tensor_t &to, const zenu_tensor_t &in, hipStream_t s)
{
    switch (fn) {
    case ZENU_EXP: return run1<T>(to, in, UnaryF<T, ZENU_EXP>(), s);
    case ZENU_LOG: return run1<T>(to, in, UnaryF<T, ZENU_LOG>(), s);
    case ZENU_TANH: return run1<T>(to, in, UnaryF<T, ZENU_TANH>(), s);
    case ZENU_SQRT: return run1<T>(to, in, UnaryF<T, ZENU_SQRT>(), s);
    case ZENU_ABS: return run1<T>(to, in, UnaryF<T, ZENU_ABS>(), s);
    case ZENU_SIGMOID: return run1<T>(to, in, UnaryF<T, ZENU_SIGMOID>(), s);
    case ZENU_TANH_ULP2:
        if constexpr (sizeof(T) == 4) return run1<T>(to, in, TanhUlp2F(), s);
        else return run1<T>(to, in, UnaryF<T, ZENU_TANH>(), s);
    default: return unary_trig(ZenuDType<T>::value, fn, to, in, s);   // ew_unary_trig.hip
    }
}

}  // namespace
}  // namespace zenu

using namespace zenu;

extern "C" {

int zenu_hip_unary(int fn, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                   zenu_stream_t stream)
{
    int rc = check2(to, other);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*to, *other)) return ZENU_ERR_SHAPE;  // "Matrix shape mismatch"
    if (dtype == ZENU_F32) return unary_t<float>(fn, *to, *other, as_stream(stream));
    if (dtype == ZENU_F64) return unary_t<double>(fn, *to, *other, as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_unary_assign(int fn, int dtype, const zenu_tensor_t *to, zenu_stream_t stream)
{
    return zenu_hip_unary(fn, dtype, to, to, stream);
}

int zenu_hip_powf(int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other, double scalar,
                  zenu_stream_t stream)
{
    int rc = check2(to, other);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (!same_shape(*to, *other)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32) { PowF<float> f; f.s = (float)scalar; return run1<float>(*to, *other, f, as_stream(stream)); }
    if (dtype == ZENU_F64) { PowF<double> f; f.s = scalar; return run1<double>(*to, *other, f, as_stream(stream)); }
    return ZENU_ERR_ARG;
}

}  // extern "C"
