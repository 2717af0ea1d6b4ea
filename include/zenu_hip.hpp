// zenu_hip.hpp -- C++17 host side over the C ABI of zenu_hip.h (header only).
//
// The reference's host side is Rust; this is the same surface for a compiled-language caller:
//   Matrix<T>      Matrix<Owned<T>/Ref<..>, DimDyn, D>      zenu-matrix/src/matrix.rs
//     views        index_axis, slice, transpose, ...        matrix.rs:347-411, shape_stride.rs:94-206
//     arithmetic   add_array / add_assign / add_scalar ...  operation/basic_operations.rs:278-381
//                  operators                                impl_ops.rs:16-254
//     unary        exp / log / tanh / ..., relu, clip        basic_operations.rs:512-575, relu.rs, clip.rs
//     reductions   sum, max_idx, max_axis, asum ...          sum.rs, max.rs, asum.rs
//     copies       copy_from, to_default_stride, broadcast  copy_from.rs, to_default_stride.rs, broadcast.rs
//   SGD / Adam / AdamW                                      zenu-optimizer/src/{sgd,adam,adamw}.rs
// Method names and argument meaning follow the reference.  Where the reference panics, Error is
// thrown with the library's status code.  Everything is one call into libzenu_hip.so on the
// current stream; nothing is computed on the host.  Buffers are owned by shared handles: a view
// keeps its buffer alive (Ref<&T> borrows in the reference), and the last owner returns the block
// to the stream-ordered pool.
#ifndef ZENU_HIP_HPP
#define ZENU_HIP_HPP

#include <cstdint>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <utility>
#include <vector>

#include "zenu_hip.h"

namespace zenu_hip {

struct Error : std::runtime_error {
    int status;
    Error(int st, const std::string &what)
        : std::runtime_error(what + ": " + zenu_hip_status_string(st) +
                             (st == ZENU_ERR_HIP ? std::string(" (") + zenu_hip_last_hip_error_string() + ")" : std::string())),
          status(st) {}
};

inline void check(int st, const char *what)
{
    if (st != ZENU_OK) throw Error(st, what);
}

inline void init(int device = 0) { check(zenu_hip_init(device), "zenu_hip_init"); }

// The stream every call of this thread of control launches on (NULL = the null stream).
inline zenu_stream_t &current_stream()
{
    static zenu_stream_t s = nullptr;
    return s;
}
inline void synchronize() { check(zenu_hip_stream_synchronize(current_stream()), "stream_synchronize"); }
// The first failure behind the reference-named void entry points of this thread since the last call
// (ZENU_OK if none); reading clears it.
inline int last_status() { return zenu_hip_last_status(); }
// After the graphs captured on `stream` are destroyed: hand the blocks their captured calls took from
// the pool back to it.
inline void release_captured(zenu_stream_t stream) { check(zenu_hip_release_captured(stream), "release_captured"); }

template <typename T> struct DType;
template <> struct DType<float> { static constexpr int value = ZENU_F32; };
template <> struct DType<double> { static constexpr int value = ZENU_F64; };

typedef std::vector<int64_t> Dim;

inline int64_t num_elm(const Dim &shape)
{
    int64_t n = 1;
    for (int64_t s : shape) n *= s;
    return n;
}

// dim/mod.rs:70-92
inline Dim default_stride(const Dim &shape)
{
    Dim st(shape.size());
    int64_t s = 1;
    for (int i = (int)shape.size() - 1; i >= 0; i--) {
        st[i] = s;
        s *= shape[i];
    }
    return st;
}

// Owned device memory (Ptr<Owned<T>, D>, matrix.rs:163-171)
// The block goes back to the pool on the stream it was taken on; a buffer that is also used on
// another stream must be kept alive until that stream is done with it.
struct Buffer {
    void *ptr = nullptr;
    size_t bytes = 0;
    zenu_stream_t stream;
    explicit Buffer(size_t n) : bytes(n), stream(current_stream()) { check(zenu_hip_malloc(&ptr, n ? n : 1, stream), "zenu_hip_malloc"); }
    ~Buffer() { if (ptr) zenu_hip_free(ptr, stream); }
    Buffer(const Buffer &) = delete;
    Buffer &operator=(const Buffer &) = delete;
};

struct Slice {   // slice_dynamic!: start..end;step (end < 0: to the end)
    int64_t start = 0, end = -1, step = 1;
    Slice() {}
    Slice(int64_t s, int64_t e, int64_t st = 1) : start(s), end(e), step(st) {}
};

template <typename T> class Matrix {
    std::shared_ptr<Buffer> buf_;
    int64_t offset_ = 0;
    Dim shape_, stride_;

    Matrix(std::shared_ptr<Buffer> b, int64_t off, Dim shape, Dim stride)
        : buf_(std::move(b)), offset_(off), shape_(std::move(shape)), stride_(std::move(stride))
    {
        if (shape_.size() > ZENU_MAX_DIM) throw std::invalid_argument("Dim must be smaller than 6");
    }
    Matrix view(int64_t off, Dim shape, Dim stride) const { return Matrix(buf_, off, std::move(shape), std::move(stride)); }
    static constexpr int dt() { return DType<T>::value; }
    static zenu_stream_t st() { return current_stream(); }

public:
    Matrix() {}

    // ---- constructors ---------------------------------------------------------------------------------
    static Matrix alloc(const Dim &shape)
    {
        return Matrix(std::make_shared<Buffer>((size_t)num_elm(shape) * sizeof(T)), 0, shape, default_stride(shape));
    }
    static Matrix zeros(const Dim &shape)
    {
        Matrix m = alloc(shape);
        check(zenu_hip_memset_zero(m.buf_->ptr, m.buf_->bytes, st()), "memset_zero");
        return m;
    }
    static Matrix from_vec(const std::vector<T> &v, const Dim &shape)
    {
        if ((int64_t)v.size() != num_elm(shape)) throw std::invalid_argument("Invalid size");
        Matrix m = alloc(shape);
        if (!v.empty()) check(zenu_hip_memcpy_h2d(m.buf_->ptr, v.data(), v.size() * sizeof(T), st()), "memcpy_h2d");
        return m;
    }
    Matrix alloc_like() const { return alloc(shape_); }
    Matrix zeros_like() const { return zeros(shape_); }

    // ---- plumbing -------------------------------------------------------------------------------------
    const Dim &shape() const { return shape_; }
    const Dim &stride() const { return stride_; }
    int64_t offset() const { return offset_; }
    int ndim() const { return (int)shape_.size(); }
    T *as_ptr() const { return static_cast<T *>(buf_->ptr) + offset_; }   // matrix.rs:288-290
    zenu_tensor_t desc() const
    {
        zenu_tensor_t t;
        t.ptr = as_ptr();
        t.ndim = ndim();
        t.reserved = 0;
        for (int i = 0; i < ZENU_MAX_DIM; i++) {
            t.shape[i] = i < ndim() ? shape_[i] : 0;
            t.stride[i] = i < ndim() ? stride_[i] : 0;
        }
        return t;
    }
    bool is_default_stride() const { return stride_ == default_stride(shape_); }
    // row-major copy of the view's elements on the host (blocking)
    std::vector<T> to_vec() const
    {
        Matrix c = is_default_stride() ? *this : to_default_stride();
        std::vector<T> v((size_t)num_elm(shape_));
        if (!v.empty()) check(zenu_hip_memcpy_d2h(v.data(), c.as_ptr(), v.size() * sizeof(T), st()), "memcpy_d2h");
        return v;
    }
    T index_item(const Dim &index) const
    {
        if (index.size() != shape_.size()) throw std::out_of_range("Index out of bounds");
        int64_t off = 0;
        for (size_t i = 0; i < index.size(); i++) {
            if (index[i] < 0 || index[i] >= shape_[i]) throw std::out_of_range("Index out of bounds");
            off += index[i] * stride_[i];
        }
        T v;
        check(zenu_hip_memcpy_d2h(&v, as_ptr() + off, sizeof(T), st()), "memcpy_d2h");
        return v;
    }

    // ---- views ----------------------------------------------------------------------------------------
    Matrix index_axis(int axis, int64_t index) const   // matrix.rs:391-403
    {
        if (axis < 0 || axis >= ndim() || index < 0 || index >= shape_[axis]) throw std::out_of_range("Index out of bounds");
        Dim sh(shape_), sd(stride_);
        sh.erase(sh.begin() + axis);
        sd.erase(sd.begin() + axis);
        return view(offset_ + stride_[axis] * index, sh, sd);
    }
    Matrix slice(const std::vector<Slice> &s) const     // matrix.rs:347-373
    {
        if ((int)s.size() > ndim()) throw std::out_of_range("too many slices");
        Dim sh(shape_), sd(stride_);
        int64_t off = offset_;
        for (size_t d = 0; d < s.size(); d++) {
            int64_t end = s[d].end < 0 || s[d].end > shape_[d] ? shape_[d] : s[d].end;
            int64_t start = s[d].start < end ? s[d].start : end;
            if (s[d].step <= 0 || start < 0) throw std::invalid_argument("bad slice");
            sh[d] = (end - start + s[d].step - 1) / s[d].step;
            sd[d] = stride_[d] * s[d].step;
            off += start * stride_[d];
        }
        return view(off, sh, sd);
    }
    Matrix transpose() const                            // shape_stride.rs:94-114
    {
        if (ndim() < 2) throw std::invalid_argument("transpose needs at least 2 dims");
        Dim sh(shape_), sd(stride_);
        std::swap(sh[ndim() - 1], sh[ndim() - 2]);
        std::swap(sd[ndim() - 1], sd[ndim() - 2]);
        return view(offset_, sh, sd);
    }
    Matrix transpose_by_index(const std::vector<int> &index) const   // shape_stride.rs:137-149
    {
        Dim sh, sd;
        for (int i : index) {
            sh.push_back(shape_.at(i));
            sd.push_back(stride_.at(i));
        }
        return view(offset_, sh, sd);
    }
    Matrix add_axis(int axis) const                     // shape_stride.rs:186-206
    {
        if (ndim() == 0) return view(offset_, {1}, {1});
        Dim sh, sd;
        for (int i = 0; i < ndim(); i++) {
            if (i == axis) {
                sh.push_back(1);
                sd.push_back(stride_[i]);
            }
            sh.push_back(shape_[i]);
            sd.push_back(stride_[i]);
        }
        if (axis == ndim()) {
            sh.push_back(1);
            sd.push_back(1);
        }
        return view(offset_, sh, sd);
    }
    Matrix reshape(const Dim &shape) const
    {
        if (num_elm(shape) != num_elm(shape_)) throw std::invalid_argument("Number of elements must be the same");
        if (!is_default_stride()) throw std::invalid_argument("reshape needs a default-stride matrix");
        return view(offset_, shape, default_stride(shape));
    }

    // ---- copies ---------------------------------------------------------------------------------------
    void copy_from(const Matrix &src) const
    {
        zenu_tensor_t a = desc(), b = src.desc();
        check(zenu_hip_copy(dt(), &a, &b, st()), "copy_from");
    }
    void broadcast(const Matrix &src) const
    {
        zenu_tensor_t a = desc(), b = src.desc();
        check(zenu_hip_broadcast(dt(), &a, &b, st()), "broadcast");
    }
    Matrix to_default_stride() const
    {
        Matrix out = alloc_like();
        out.copy_from(*this);
        return out;
    }
    Matrix new_matrix() const { return to_default_stride(); }

    // ---- arithmetic -----------------------------------------------------------------------------------
    void binary_array(int op, const Matrix &lhs, const Matrix &rhs) const
    {
        zenu_tensor_t t = desc(), l = lhs.desc(), r = rhs.desc();
        check(zenu_hip_binary(op, dt(), &t, &l, &r, st()), "array_array");
    }
    void binary_assign(int op, const Matrix &rhs) const
    {
        zenu_tensor_t t = desc(), r = rhs.desc();
        check(zenu_hip_binary_assign(op, dt(), &t, &r, st()), "array_assign");
    }
    void binary_scalar(int op, const Matrix &other, T s) const
    {
        zenu_tensor_t t = desc(), o = other.desc();
        check(zenu_hip_binary_scalar(op, dt(), &t, &o, (double)s, st()), "scalar");
    }
    void binary_scalar_assign(int op, T s) const
    {
        zenu_tensor_t t = desc();
        check(zenu_hip_binary_scalar_assign(op, dt(), &t, (double)s, st()), "scalar_assign");
    }
#define ZENU_HPP_NAMED(name, OP)                                                                   \
    void name##_array(const Matrix &l, const Matrix &r) const { binary_array(OP, l, r); }          \
    void name##_assign(const Matrix &r) const { binary_assign(OP, r); }                            \
    void name##_scalar(const Matrix &o, T s) const { binary_scalar(OP, o, s); }                    \
    void name##_scalar_assign(T s) const { binary_scalar_assign(OP, s); }
    ZENU_HPP_NAMED(add, ZENU_ADD)
    ZENU_HPP_NAMED(sub, ZENU_SUB)
    ZENU_HPP_NAMED(mul, ZENU_MUL)
    ZENU_HPP_NAMED(div, ZENU_DIV)
#undef ZENU_HPP_NAMED

    // impl_ops.rs:16-254: the output takes the larger operand's shape; a 0-d operand is a
    // device-side scalar (scalar_ptr, basic_operations.rs:74-88)
    Matrix operate(int op, const Matrix &rhs) const
    {
        if (rhs.ndim() == 0 && ndim() > 0) {
            Matrix out = alloc_like();
            zenu_tensor_t t = out.desc(), o = desc();
            check(zenu_hip_binary_scalar_ptr(op, dt(), &t, &o, rhs.as_ptr(), st()), "scalar_ptr");
            return out;
        }
        const Matrix &big = (num_elm(rhs.shape_) > num_elm(shape_) || rhs.ndim() > ndim()) ? rhs : *this;
        Matrix out = alloc(big.shape_);
        out.binary_array(op, *this, rhs);
        return out;
    }
    Matrix operator+(const Matrix &r) const { return operate(ZENU_ADD, r); }
    Matrix operator-(const Matrix &r) const { return operate(ZENU_SUB, r); }
    Matrix operator*(const Matrix &r) const { return operate(ZENU_MUL, r); }
    Matrix operator/(const Matrix &r) const { return operate(ZENU_DIV, r); }
    Matrix scalar_op(int op, T s) const
    {
        Matrix out = alloc_like();
        out.binary_scalar(op, *this, s);
        return out;
    }
    Matrix operator+(T s) const { return scalar_op(ZENU_ADD, s); }
    Matrix operator-(T s) const { return scalar_op(ZENU_SUB, s); }
    Matrix operator*(T s) const { return scalar_op(ZENU_MUL, s); }
    Matrix operator/(T s) const { return scalar_op(ZENU_DIV, s); }
    const Matrix &operator+=(const Matrix &r) const { binary_assign(ZENU_ADD, r); return *this; }
    const Matrix &operator-=(const Matrix &r) const { binary_assign(ZENU_SUB, r); return *this; }
    const Matrix &operator*=(const Matrix &r) const { binary_assign(ZENU_MUL, r); return *this; }
    const Matrix &operator/=(const Matrix &r) const { binary_assign(ZENU_DIV, r); return *this; }

    // ---- unary ----------------------------------------------------------------------------------------
    void unary_array(int fn, const Matrix &other) const
    {
        zenu_tensor_t t = desc(), o = other.desc();
        check(zenu_hip_unary(fn, dt(), &t, &o, st()), "unary");
    }
    void unary_assign(int fn) const
    {
        zenu_tensor_t t = desc();
        check(zenu_hip_unary_assign(fn, dt(), &t, st()), "unary_assign");
    }
    Matrix unary(int fn) const
    {
        Matrix out = alloc_like();
        out.unary_array(fn, *this);
        return out;
    }
#define ZENU_HPP_UNARY(name, FN)                                                                   \
    Matrix name() const { return unary(FN); }                                                      \
    void name##_array(const Matrix &o) const { unary_array(FN, o); }                               \
    void name##_assign() const { unary_assign(FN); }
    ZENU_HPP_UNARY(exp, ZENU_EXP)
    ZENU_HPP_UNARY(log, ZENU_LOG)
    ZENU_HPP_UNARY(tanh, ZENU_TANH)
    ZENU_HPP_UNARY(sqrt, ZENU_SQRT)
    ZENU_HPP_UNARY(abs, ZENU_ABS)
    ZENU_HPP_UNARY(sin, ZENU_SIN)
    ZENU_HPP_UNARY(cos, ZENU_COS)
    ZENU_HPP_UNARY(tan, ZENU_TAN)
    ZENU_HPP_UNARY(asin, ZENU_ASIN)
    ZENU_HPP_UNARY(acos, ZENU_ACOS)
    ZENU_HPP_UNARY(atan, ZENU_ATAN)
    ZENU_HPP_UNARY(sinh, ZENU_SINH)
    ZENU_HPP_UNARY(cosh, ZENU_COSH)
    ZENU_HPP_UNARY(sigmoid, ZENU_SIGMOID)
    ZENU_HPP_UNARY(tanh_ulp2, ZENU_TANH_ULP2)   // not in the reference: f32 tanh within 2 ulp of tanh(), memory-bound
#undef ZENU_HPP_UNARY
    void powf(const Matrix &other, T s) const
    {
        zenu_tensor_t t = desc(), o = other.desc();
        check(zenu_hip_powf(dt(), &t, &o, (double)s, st()), "powf");
    }
    void relu(const Matrix &other, T alpha) const
    {
        zenu_tensor_t t = desc(), o = other.desc();
        check(zenu_hip_relu(dt(), &t, &o, (double)alpha, st()), "relu");
    }
    void relu_backward_mask(const Matrix &other, T alpha) const
    {
        zenu_tensor_t t = desc(), o = other.desc();
        check(zenu_hip_relu_backward_mask(dt(), &t, &o, (double)alpha, st()), "relu_backward_mask");
    }
    void relu_backward(const Matrix &gy, const Matrix &x, T alpha) const
    {
        zenu_tensor_t t = desc(), g = gy.desc(), xx = x.desc();
        check(zenu_hip_relu_backward(dt(), &t, &g, &xx, (double)alpha, st()), "relu_backward");
    }
    // *this = gy * relu'(x) and gbias = its column sums (the bias gradient of the layer before), one pass
    void relu_backward_bias_grad(const Matrix &gbias, const Matrix &gy, const Matrix &x, T alpha) const
    {
        zenu_tensor_t t = desc(), b = gbias.desc(), g = gy.desc(), xx = x.desc();
        check(zenu_hip_relu_backward_bias_grad(dt(), &t, &b, &g, &xx, (double)alpha, st()), "relu_backward_bias_grad");
    }
    void tanh_backward(const Matrix &gy, const Matrix &x) const      // functions/tanh.rs:30-37
    {
        zenu_tensor_t t = desc(), g = gy.desc(), xx = x.desc();
        check(zenu_hip_tanh_backward(dt(), &t, &g, &xx, st()), "tanh_backward");
    }
    void sigmoid_backward(const Matrix &gy, const Matrix &x) const   // activation/sigmoid.rs:7-15
    {
        zenu_tensor_t t = desc(), g = gy.desc(), xx = x.desc();
        check(zenu_hip_sigmoid_backward(dt(), &t, &g, &xx, st()), "sigmoid_backward");
    }
    Matrix clip(T lo, T hi) const
    {
        Matrix out = alloc_like();
        zenu_tensor_t t = out.desc(), o = desc();
        check(zenu_hip_clip(dt(), &t, &o, (double)lo, (double)hi, st()), "clip");
        return out;
    }
    void clip_assign(T lo, T hi) const
    {
        zenu_tensor_t t = desc();
        check(zenu_hip_clip(dt(), &t, &t, (double)lo, (double)hi, st()), "clip_assign");
    }
    Matrix clip_backward_mask(T lo, T hi) const
    {
        Matrix out = alloc_like();
        zenu_tensor_t t = out.desc(), o = desc();
        check(zenu_hip_clip_backward_mask(dt(), &t, &o, (double)lo, (double)hi, st()), "clip_backward_mask");
        return out;
    }
    void softmax_assign(const Matrix &src, int axis) const
    {
        if (axis < 0 || axis >= ndim()) throw Error(ZENU_ERR_AXIS, "axis must be less than the number of dimensions");
        zenu_tensor_t t = desc(), s = src.desc();
        check(zenu_hip_softmax(dt(), &t, &s, axis, st()), "softmax_assign");
    }
    void bias_add_relu(const Matrix &z, const Matrix &bias, T alpha, const Matrix *pre = nullptr) const
    {
        zenu_tensor_t t = desc(), zz = z.desc(), b = bias.desc(), p;
        if (pre) p = pre->desc();
        check(zenu_hip_bias_add_relu(dt(), pre ? &p : nullptr, &t, &zz, &b, (double)alpha, st()), "bias_add_relu");
    }

    // ---- reductions -----------------------------------------------------------------------------------
    Matrix sum(int axis, bool keep_dim = false) const     // sum.rs:9-32
    {
        if (axis < 0 || axis >= ndim()) throw Error(ZENU_ERR_AXIS, "Invalid axis");
        Dim sh(shape_);
        sh.erase(sh.begin() + axis);
        Matrix out = alloc(sh);
        zenu_tensor_t o = out.desc(), s = desc();
        check(zenu_hip_sum_axis(dt(), &o, &s, axis, st()), "sum");
        return keep_dim ? out.add_axis(axis) : out;
    }
    // the same sum into an existing `out` through the entry point that allocates nothing (for callers that
    // cannot allocate: its scratch is a fixed device array, see zenu_hip.h for the limits)
    void sum_noalloc(int axis, const Matrix &out) const
    {
        zenu_tensor_t o = out.desc(), s = desc();
        check(zenu_hip_sum_axis_noalloc(dt(), &o, &s, axis, st()), "sum_noalloc");
    }
    Matrix sum_all() const
    {
        Matrix out = alloc({});
        zenu_tensor_t s = desc();
        check(zenu_hip_sum_all(dt(), out.as_ptr(), &s, st()), "sum_all");
        return out;
    }
    void sum_to(const Matrix &target) const               // target = sum_to(self), sum.rs:35-94
    {
        zenu_tensor_t t = target.desc(), s = desc();
        check(zenu_hip_sum_to(dt(), &t, &s, st()), "sum_to");
    }
    Matrix max_axis(int axis, bool keep_dim = false) const   // max.rs:67-99
    {
        if (axis < 0 || axis >= ndim()) throw Error(ZENU_ERR_AXIS, "Invalid axis");
        Dim sh(shape_);
        sh.erase(sh.begin() + axis);
        Matrix out = alloc(sh);
        zenu_tensor_t o = out.desc(), s = desc();
        check(zenu_hip_max_axis(dt(), &o, &s, axis, st()), "max_axis");
        return keep_dim ? out.add_axis(axis) : out;
    }
    std::vector<int64_t> max_axis_idx_ravel(int axis) const  // max.rs:103-134
    {
        if (axis < 0 || axis >= ndim()) throw Error(ZENU_ERR_AXIS, "Invalid axis");
        const int64_t n = shape_[axis] ? num_elm(shape_) / shape_[axis] : 0;
        Buffer idx((size_t)n * sizeof(int64_t));
        zenu_tensor_t s = desc();
        check(zenu_hip_max_axis_idx(dt(), static_cast<int64_t *>(idx.ptr), &s, axis, st()), "max_axis_idx");
        std::vector<int64_t> out((size_t)n);
        if (n) check(zenu_hip_memcpy_d2h(out.data(), idx.ptr, out.size() * sizeof(int64_t), st()), "memcpy_d2h");
        return out;
    }
    Dim max_idx() const                                   // max.rs:45-56: N-d index of the first maximum
    {
        Buffer idx(sizeof(int64_t));
        zenu_tensor_t s = desc();
        check(zenu_hip_max_idx(dt(), static_cast<int64_t *>(idx.ptr), nullptr, &s, st()), "max_idx");
        int64_t flat = 0;
        check(zenu_hip_memcpy_d2h(&flat, idx.ptr, sizeof flat, st()), "memcpy_d2h");
        Dim out(shape_.size());
        for (int i = ndim() - 1; i >= 0; i--) {
            out[i] = flat % shape_[i];
            flat /= shape_[i];
        }
        return out;
    }
    T max_item() const                                    // max.rs:59-62
    {
        Buffer idx(sizeof(int64_t)), val(sizeof(T));
        zenu_tensor_t s = desc();
        check(zenu_hip_max_idx(dt(), static_cast<int64_t *>(idx.ptr), val.ptr, &s, st()), "max_item");
        T v;
        check(zenu_hip_memcpy_d2h(&v, val.ptr, sizeof v, st()), "memcpy_d2h");
        return v;
    }
    Matrix mean(int axis, bool keep_dim = false) const    // mean.rs:10-13
    {
        return sum(axis, keep_dim) / (T)shape()[axis];
    }
    Matrix mean_all() const                               // mean.rs:15-19: asum / num_elm, the mean of |x|
    {
        return from_vec({asum() / (T)num_elm(shape())}, {});
    }
    Matrix variance(int axis, bool keep_dim = false) const   // var.rs:19-26
    {
        Matrix diff = *this - mean(axis, true);
        return (diff * diff).mean(axis, keep_dim);
    }
    Matrix variance_all() const
    {
        Matrix diff = *this - mean_all();
        return (diff * diff).mean_all();
    }
    T asum() const                                        // asum.rs:49-68
    {
        Buffer val(sizeof(T));
        zenu_tensor_t s = desc();
        check(zenu_hip_asum(dt(), val.ptr, &s, st()), "asum");
        T v;
        check(zenu_hip_memcpy_d2h(&v, val.ptr, sizeof v, st()), "memcpy_d2h");
        return v;
    }
};

// ---- fused loss chains (zenu-autograd/src/loss/{softmax,cross_entropy}.rs) -------------------------------------

template <typename T> Matrix<T> softmax_backward(const Matrix<T> &y, const Matrix<T> &gy, int axis)
{
    Matrix<T> gx = y.alloc_like();
    zenu_tensor_t g = gx.desc(), yy = y.desc(), gg = gy.desc();
    check(zenu_hip_softmax_backward(DType<T>::value, &g, &yy, &gg, axis, current_stream()), "softmax_backward");
    return gx;
}

// (loss, prob) of cross_entropy(pred, ans)
template <typename T> std::pair<Matrix<T>, Matrix<T>> cross_entropy(const Matrix<T> &pred, const Matrix<T> &ans)
{
    Matrix<T> loss = Matrix<T>::alloc({}), prob = pred.alloc_like();
    zenu_tensor_t l = loss.desc(), p = prob.desc(), x = pred.desc(), a = ans.desc();
    check(zenu_hip_softmax_cross_entropy(DType<T>::value, &l, &p, &x, &a, current_stream()), "cross_entropy");
    return {loss, prob};
}

template <typename T>
Matrix<T> cross_entropy_backward(const Matrix<T> &prob, const Matrix<T> &ans, const Matrix<T> *gloss = nullptr)
{
    Matrix<T> g = prob.alloc_like();
    zenu_tensor_t gd = g.desc(), p = prob.desc(), a = ans.desc(), gl;
    if (gloss) gl = gloss->desc();
    check(zenu_hip_softmax_cross_entropy_backward(DType<T>::value, &gd, &p, &a, gloss ? &gl : nullptr, current_stream()),
          "cross_entropy_backward");
    return g;
}

// cross_entropy_backward that also writes the column sums of the gradient (the bias gradient of the
// layer that produced the logits) to gbias
template <typename T>
Matrix<T> cross_entropy_backward_bias_grad(const Matrix<T> &prob, const Matrix<T> &ans, const Matrix<T> &gbias,
                                           const Matrix<T> *gloss = nullptr)
{
    Matrix<T> g = prob.alloc_like();
    zenu_tensor_t gd = g.desc(), b = gbias.desc(), p = prob.desc(), a = ans.desc(), gl;
    if (gloss) gl = gloss->desc();
    check(zenu_hip_softmax_cross_entropy_backward_bias_grad(DType<T>::value, &gd, &b, &p, &a, gloss ? &gl : nullptr,
                                                            current_stream()),
          "cross_entropy_backward_bias_grad");
    return g;
}

// ---- stack / split (zenu-matrix/src/operation/stack.rs:18-58, split.rs:20-58): one strided copy per piece ------

template <typename T> Matrix<T> axis_range(const Matrix<T> &m, int axis, int64_t start, int64_t stop)
{
    std::vector<Slice> s((size_t)axis + 1);
    s[(size_t)axis] = Slice(start, stop);
    return m.slice(s);
}

template <typename T> Matrix<T> stack(const std::vector<Matrix<T>> &matrices, int axis)
{
    if (matrices.empty()) throw Error(ZENU_ERR_ARG, "stack: No matrices to stack");
    const Dim first = matrices[0].shape();
    for (const Matrix<T> &m : matrices)
        if (m.shape() != first) throw Error(ZENU_ERR_SHAPE, "stack: All matrices must have the same shape");
    if (axis < 0 || axis >= (int)first.size()) throw Error(ZENU_ERR_AXIS, "stack");
    const int64_t n = first[(size_t)axis];
    Dim shape = first;
    shape[(size_t)axis] = n * (int64_t)matrices.size();
    Matrix<T> out = Matrix<T>::alloc(shape);
    for (size_t i = 0; i < matrices.size(); i++) axis_range(out, axis, (int64_t)i * n, (int64_t)(i + 1) * n).copy_from(matrices[i]);
    return out;
}

template <typename T> std::vector<Matrix<T>> split(const Matrix<T> &matrix, int axis, int num_splits)
{
    if (axis < 0 || axis >= matrix.ndim()) throw Error(ZENU_ERR_AXIS, "split");
    if (num_splits <= 0 || matrix.shape()[(size_t)axis] % num_splits) throw Error(ZENU_ERR_SHAPE, "split");
    const int64_t n = matrix.shape()[(size_t)axis] / num_splits;
    Dim shape = matrix.shape();
    shape[(size_t)axis] = n;
    std::vector<Matrix<T>> outs;
    for (int i = 0; i < num_splits; i++) {
        Matrix<T> o = Matrix<T>::alloc(shape);
        o.copy_from(axis_range(matrix, axis, (int64_t)i * n, (int64_t)(i + 1) * n));
        outs.push_back(o);
    }
    return outs;
}

// ---- ConvBias (zenu-matrix/src/nn/conv/mod.rs:84-107; the CPU device's definitions, cpu/bias.rs) ----------------

template <typename T> bool is_channel_bias(const Matrix<T> &bias, const Matrix<T> &x)
{
    const Dim &b = bias.shape(), &s = x.shape();
    return b.size() == 4 && s.size() == 4 && b[0] == 1 && b[2] == 1 && b[3] == 1 && b[1] == s[1];
}

// output[N,C,H,W] = input + bias[1,C,1,1]
template <typename T> void conv2d_bias_add(const Matrix<T> &input, const Matrix<T> &bias, const Matrix<T> &output)
{
    if (input.shape() != output.shape() || !is_channel_bias(bias, output)) throw Error(ZENU_ERR_SHAPE, "conv2d_bias_add");
    output.add_array(input, bias);
}

// d_bias[1,C,1,1] = d_output summed over axes 0, 2 and 3
template <typename T> void conv2d_bias_bkwd(const Matrix<T> &d_output, const Matrix<T> &d_bias)
{
    if (!is_channel_bias(d_bias, d_output)) throw Error(ZENU_ERR_SHAPE, "conv2d_bias_bkwd");
    d_output.sum_to(d_bias);
}

// ---- optimizers: name -> (parameter, gradient); a default-constructed gradient means "no grad" -----------------

template <typename T> struct ParamGrad {
    Matrix<T> data, grad;
    bool has_grad = false;
    ParamGrad() {}
    ParamGrad(Matrix<T> d) : data(std::move(d)) {}
    ParamGrad(Matrix<T> d, Matrix<T> g) : data(std::move(d)), grad(std::move(g)), has_grad(true) {}
};
template <typename T> using Parameters = std::map<std::string, ParamGrad<T>>;

template <typename T> class SGD {           // zenu-optimizer/src/sgd.rs:6-31
public:
    T learning_rate;
    explicit SGD(T lr) : learning_rate(lr) {}
    void update(const Parameters<T> &params) const        // one launch for all tensors
    {
        std::vector<void *> p;
        std::vector<const void *> g;
        std::vector<int64_t> n;
        for (const auto &kv : params) {
            const ParamGrad<T> &pg = kv.second;
            if (!pg.has_grad) continue;
            if (!pg.data.is_default_stride() || !pg.grad.is_default_stride()) throw std::invalid_argument("optimizer tensors must be default stride");
            p.push_back(pg.data.as_ptr());
            g.push_back(pg.grad.as_ptr());
            n.push_back(num_elm(pg.data.shape()));
        }
        if (p.empty()) return;
        check(zenu_hip_sgd_step_multi(DType<T>::value, (int)p.size(), p.data(), g.data(), n.data(), (double)learning_rate,
                                      current_stream()), "sgd_step_multi");
    }
};

template <typename T> class AdamW {         // zenu-optimizer/src/adamw.rs:9-101; weight_decay 0 and no weights = Adam
public:
    T learning_rate, beta1, beta2, epsilon, weight_decay;
    int64_t step = 0;
    std::map<std::string, Matrix<T>> m, v;
    std::set<std::string> weight_keys;

    AdamW(T lr, T b1, T b2, T eps, T wd, const Parameters<T> &params, std::set<std::string> weights = {})
        : learning_rate(lr), beta1(b1), beta2(b2), epsilon(eps), weight_decay(wd), weight_keys(std::move(weights))
    {
        for (const auto &kv : params) {     // zeros_like per parameter (adam.rs:62-88)
            m.emplace(kv.first, kv.second.data.zeros_like());
            v.emplace(kv.first, kv.second.data.zeros_like());
        }
    }

    ~AdamW() { drop_schedule(); }
    AdamW(const AdamW &) = delete;
    AdamW &operator=(const AdamW &) = delete;

    // For callers that record `update` into a HIP graph: take 1 - beta^t of the next n_steps updates from
    // a table in device memory whose cursor every update advances, so that each replay of one recorded
    // update is the next step (zenu_hip_adam_step_multi_scheduled; no counterpart in the reference).
    void use_schedule(int n_steps)
    {
        drop_schedule();
        check(zenu_hip_adam_schedule_create(&schedule_, DType<T>::value, (double)beta1, (double)beta2, step + 1, n_steps,
                                            current_stream()), "adam_schedule_create");
    }
    void drop_schedule()
    {
        if (schedule_) zenu_hip_adam_schedule_destroy(schedule_, current_stream());
        schedule_ = nullptr;
    }
    // next step of the schedule, steps left in it, updates refused because it had run out
    void schedule_state(int64_t &next_step, int64_t &steps_left, int64_t &refused) const
    {
        check(zenu_hip_adam_schedule_query(schedule_, &next_step, &steps_left, &refused, current_stream()), "adam_schedule_query");
    }

    // one launch for the whole model (zenu_hip_adam_step_multi)
    void update(const Parameters<T> &params)
    {
        step += 1;
        std::vector<void *> P, M, V;
        std::vector<const void *> G;
        std::vector<int64_t> sizes;
        std::vector<int32_t> decay;
        for (const auto &kv : params) {
            const ParamGrad<T> &pg = kv.second;
            if (!pg.has_grad) continue;
            const Matrix<T> &mm = m.at(kv.first), &vv = v.at(kv.first);
            if (!pg.data.is_default_stride() || !pg.grad.is_default_stride()) throw std::invalid_argument("optimizer tensors must be default stride");
            P.push_back(pg.data.as_ptr());
            G.push_back(pg.grad.as_ptr());
            M.push_back(mm.as_ptr());
            V.push_back(vv.as_ptr());
            sizes.push_back(num_elm(pg.data.shape()));
            decay.push_back(weight_keys.count(kv.first) ? 1 : 0);
        }
        if (P.empty()) return;
        if (schedule_) {
            check(zenu_hip_adam_step_multi_scheduled(DType<T>::value, (int)P.size(), P.data(), G.data(), M.data(), V.data(),
                                                     sizes.data(), (double)learning_rate, (double)epsilon, (double)weight_decay,
                                                     decay.data(), schedule_, current_stream()),
                  "adam_step_multi_scheduled");
            return;
        }
        check(zenu_hip_adam_step_multi(DType<T>::value, (int)P.size(), P.data(), G.data(), M.data(), V.data(), sizes.data(),
                                       (double)learning_rate, (double)beta1, (double)beta2, (double)epsilon,
                                       (double)weight_decay, decay.data(), (double)step, current_stream()),
              "adam_step_multi");
    }

private:
    void *schedule_ = nullptr;
};

template <typename T> class Adam : public AdamW<T> {   // zenu-optimizer/src/adam.rs:9-89
public:
    Adam(T lr, T b1, T b2, T eps, const Parameters<T> &params) : AdamW<T>(lr, b1, b2, eps, (T)0, params) {}
};

}  // namespace zenu_hip

#endif  // ZENU_HIP_HPP
