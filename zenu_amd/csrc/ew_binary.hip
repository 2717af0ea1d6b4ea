// ew_binary.hip -- entry points of the array-array and array-scalar operators
// (zenu-matrix/src/operation/basic_operations.rs:278-381); engine in elementwise.hpp.
#include "elementwise.hpp"

namespace zenu {
namespace {

template <typename T> int binary_t(int op, const zenu_tensor_t &to, const zenu_tensor_t &l,
                                   const zenu_tensor_t &r, hipStream_t s)
{
    switch (op) {
    case ZENU_ADD: return run2<T>(to, l, r, BinF<T, ZENU_ADD>(), s);
    case ZENU_SUB: return run2<T>(to, l, r, BinF<T, ZENU_SUB>(), s);
    case ZENU_MUL: return run2<T>(to, l, r, BinF<T, ZENU_MUL>(), s);
    case ZENU_DIV: return run2<T>(to, l, r, BinF<T, ZENU_DIV>(), s);
    default: return ZENU_ERR_ARG;
    }
}

template <typename T> int scalar_t(int op, const zenu_tensor_t &to, const zenu_tensor_t &in, T sv,
                                   const T *sp, hipStream_t s)
{
    switch (op) {
    case ZENU_ADD: { ScalarF<T, ZENU_ADD> f; f.s = sv; f.sp = sp; return run1<T>(to, in, f, s); }
    case ZENU_SUB: { ScalarF<T, ZENU_SUB> f; f.s = sv; f.sp = sp; return run1<T>(to, in, f, s); }
    case ZENU_MUL: { ScalarF<T, ZENU_MUL> f; f.s = sv; f.sp = sp; return run1<T>(to, in, f, s); }
    case ZENU_DIV: { ScalarF<T, ZENU_DIV> f; f.s = sv; f.sp = sp; return run1<T>(to, in, f, s); }
    default: return ZENU_ERR_ARG;
    }
}

}  // namespace
}  // namespace zenu

using namespace zenu;

extern "C" {

int zenu_hip_binary(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *lhs,
                    const zenu_tensor_t *rhs, zenu_stream_t stream)
{
    int rc = check2(to, lhs);
    if (!rc) rc = validate_tensor(rhs);
    if (!rc) rc = ensure_init();
    if (!rc) rc = check_binary(*to, *lhs, *rhs);
    if (rc) return rc;
    if (dtype == ZENU_F32) return binary_t<float>(op, *to, *lhs, *rhs, as_stream(stream));
    if (dtype == ZENU_F64) return binary_t<double>(op, *to, *lhs, *rhs, as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_binary_assign(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *rhs,
                           zenu_stream_t stream)
{
    int rc = check2(to, rhs);
    if (!rc) rc = ensure_init();
    if (!rc) rc = check_binary_assign(*to, *rhs);
    if (rc) return rc;
    if (dtype == ZENU_F32) return binary_t<float>(op, *to, *to, *rhs, as_stream(stream));
    if (dtype == ZENU_F64) return binary_t<double>(op, *to, *to, *rhs, as_stream(stream));
    return ZENU_ERR_ARG;
}

static int scalar_common(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                         double scalar, const void *sp, zenu_stream_t stream)
{
    int rc = check2(to, other);
    if (!rc) rc = ensure_init();
    if (rc) return rc;
    if (to->ndim < other->ndim) return ZENU_ERR_RANK;   // with_clousers.rs:42-50
    if (!same_shape(*to, *other)) return ZENU_ERR_SHAPE;
    if (dtype == ZENU_F32)
        return scalar_t<float>(op, *to, *other, (float)scalar, static_cast<const float *>(sp),
                               as_stream(stream));
    if (dtype == ZENU_F64)
        return scalar_t<double>(op, *to, *other, scalar, static_cast<const double *>(sp),
                                as_stream(stream));
    return ZENU_ERR_ARG;
}

int zenu_hip_binary_scalar(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                           double scalar, zenu_stream_t stream)
{
    return scalar_common(op, dtype, to, other, scalar, nullptr, stream);
}

int zenu_hip_binary_scalar_assign(int op, int dtype, const zenu_tensor_t *to, double scalar,
                                  zenu_stream_t stream)
{
    return scalar_common(op, dtype, to, to, scalar, nullptr, stream);
}

int zenu_hip_binary_scalar_ptr(int op, int dtype, const zenu_tensor_t *to, const zenu_tensor_t *other,
                               const void *scalar_dev, zenu_stream_t stream)
{
    if (!scalar_dev) return ZENU_ERR_ARG;
    return scalar_common(op, dtype, to, other, 0.0, scalar_dev, stream);
}

int zenu_hip_binary_scalar_assign_ptr(int op, int dtype, const zenu_tensor_t *to,
                                      const void *scalar_dev, zenu_stream_t stream)
{
    if (!scalar_dev) return ZENU_ERR_ARG;
    return scalar_common(op, dtype, to, to, 0.0, scalar_dev, stream);
}

}  // extern "C"
