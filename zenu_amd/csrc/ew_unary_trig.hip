// ew_unary_trig.hip -- sin, cos, tan, asin, acos, atan, sinh, cosh (basic_operations.rs:441-510)
// behind zenu_hip_unary; engine in elementwise.hpp.
#include "elementwise.hpp"

namespace zenu {
namespace {

template <typename T> int unary_trig_t(int fn, const zenu_tensor_t &to, const zenu_tensor_t &in, hipStream_t s)
{
    switch (fn) {
    case ZENU_SIN: return run1<T>(to, in, UnaryF<T, ZENU_SIN>(), s);
    case ZENU_COS: return run1<T>(to, in, UnaryF<T, ZENU_COS>(), s);
    case ZENU_TAN: return run1<T>(to, in, UnaryF<T, ZENU_TAN>(), s);
    case ZENU_ASIN: return run1<T>(to, in, UnaryF<T, ZENU_ASIN>(), s);
    case ZENU_ACOS: return run1<T>(to, in, UnaryF<T, ZENU_ACOS>(), s);
    case ZENU_ATAN: return run1<T>(to, in, UnaryF<T, ZENU_ATAN>(), s);
    case ZENU_SINH: return run1<T>(to, in, UnaryF<T, ZENU_SINH>(), s);
    case ZENU_COSH: return run1<T>(to, in, UnaryF<T, ZENU_COSH>(), s);
    default: return ZENU_ERR_ARG;
    }
}

}  // namespace

int unary_trig(int dtype, int fn, const zenu_tensor_t &to, const zenu_tensor_t &in, hipStream_t s)
{
    if (dtype == ZENU_F32) return unary_trig_t<float>(fn, to, in, s);
    if (dtype == ZENU_F64) return unary_trig_t<double>(fn, to, in, s);
    return ZENU_ERR_ARG;
}

}  // namespace zenu
