"""Host-side mirror of zenu-matrix's `Matrix` for the HIP device, on top of the C ABI.

The method names, argument meaning and error behaviour follow the reference so that parity
tests read like the reference's own tests:

  constructors  from_vec / zeros / alloc            zenu-matrix/src/constructor/*.rs
  views         index_axis / slice / transpose ...  zenu-matrix/src/matrix.rs:347-411,
                                                    zenu-matrix/src/shape_stride.rs:94-114
  arithmetic    add_array, add_assign, add_scalar, add_scalar_assign (+ sub/mul/div) and the
                operators                           zenu-matrix/src/operation/basic_operations.rs:278-381,
                                                    zenu-matrix/src/impl_ops.rs:16-254
  unary         exp/log/tanh/sqrt/abs ..., relu     basic_operations.rs:512-575, relu.rs:169-242
  reductions    sum, sum_to, max_idx, max_item, max_axis, max_axis_idx_ravel, asum
                                                    sum.rs:9-94, max.rs:43-135, asum.rs:49-68
  copies        copy_from, to_default_stride        copy_from.rs:211-267, to_default_stride.rs:7-15

Where the reference panics, a ZenuHipError is raised (status RANK / SHAPE / AXIS).  Every
operation is one call into libzenu_hip.so; nothing here computes on the host.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import ZenuHipError, Tensor, check

_stream = None  # hipStream_t as int / None = null stream


def set_stream(stream):
    global _stream
    _stream = stream


def get_stream():
    return _stream


def synchronize():
    check(_lib.lib().zenu_hip_stream_synchronize(_stream), "stream_synchronize")


def _dt(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return _lib.F32
    if dtype == np.float64:
        return _lib.F64
    raise TypeError(f"unsupported dtype {dtype}")


def default_stride(shape):
    """zenu-matrix/src/dim/mod.rs:70-92"""
    stride = [1] * len(shape)
    for i in range(len(shape) - 2, -1, -1):
        stride[i] = stride[i + 1] * shape[i + 1]
    return tuple(stride)


class DeviceBuffer:
    """Owned device memory (Ptr<Owned<T>, D>): freed through the pool when dropped
    (zenu-matrix/src/matrix.rs:163-171)."""

    def __init__(self, nbytes):
        p = C.c_void_p()
        # the block is returned on the stream it was taken on: a buffer used on another stream
        # as well must be kept alive until that stream is done with it
        self.stream = _stream
        check(_lib.lib().zenu_hip_malloc(C.byref(p), nbytes, self.stream), "malloc")
        self.ptr = p.value
        self.nbytes = nbytes

    def __del__(self):
        try:
            if getattr(self, "ptr", None):
                _lib.lib().zenu_hip_free(self.ptr, self.stream)
                self.ptr = None
        except Exception:
            pass


class Matrix:
    def __init__(self, buf, offset, shape, stride, dtype):
        self.buf = buf
        self.offset = int(offset)
        self.shape = tuple(int(s) for s in shape)
        self.stride = tuple(int(s) for s in stride)
        self.dtype = np.dtype(dtype)
        if len(self.shape) > _lib.MAX_DIM:
            raise ValueError("Dim must be smaller than 6")

    # ---- constructors -------------------------------------------------------------------
    @staticmethod
    def alloc(shape, dtype=np.float32):
        shape = tuple(shape)
        n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
        dtype = np.dtype(dtype)
        return Matrix(DeviceBuffer(max(n, 1) * dtype.itemsize), 0, shape, default_stride(shape), dtype)

    @staticmethod
    def zeros(shape, dtype=np.float32):
        m = Matrix.alloc(shape, dtype)
        check(_lib.lib().zenu_hip_memset_zero(m.buf.ptr, m.buf.nbytes, _stream), "memset_zero")
        return m

    @staticmethod
    def from_numpy(arr):
        arr = np.asarray(arr)
        if not arr.flags["C_CONTIGUOUS"]:
            arr = arr.copy(order="C")
        m = Matrix.alloc(arr.shape, arr.dtype)
        if arr.size:
            check(_lib.lib().zenu_hip_memcpy_h2d(m.buf.ptr, arr.ctypes.data, arr.nbytes, _stream), "h2d")
        return m

    @staticmethod
    def from_vec(vec, shape, dtype=np.float32):
        return Matrix.from_numpy(np.asarray(vec, dtype=dtype).reshape(tuple(shape)))

    def alloc_like(self):
        return Matrix.alloc(self.shape, self.dtype)

    # ---- plumbing -----------------------------------------------------------------------
    @property
    def ndim(self):
        return len(self.shape)

    def num_elm(self):
        return int(np.prod(self.shape, dtype=np.int64)) if self.shape else 1

    def as_ptr(self):
        """matrix.rs:288-290"""
        return self.buf.ptr + self.offset * self.dtype.itemsize

    def desc(self):
        t = Tensor()
        t.ptr = self.as_ptr()
        t.ndim = self.ndim
        for i in range(self.ndim):
            t.shape[i] = self.shape[i]
            t.stride[i] = self.stride[i]
        return t

    def _view(self, offset, shape, stride):
        return Matrix(self.buf, offset, shape, stride, self.dtype)

    def to_numpy(self):
        src = self if self.is_default_stride_strict() else self.to_default_stride()
        out = np.empty(self.shape, dtype=self.dtype)
        if out.size:
            check(_lib.lib().zenu_hip_memcpy_d2h(out.ctypes.data, src.as_ptr(), out.nbytes, _stream), "d2h")
        return out

    def is_default_stride_strict(self):
        return self.stride == default_stride(self.shape)

    def is_default_stride(self):
        """shape_stride.rs:116-121"""
        return self.ndim == 1 or self.is_default_stride_strict()

    # ---- views --------------------------------------------------------------------------
    def index_axis(self, axis, index):
        """matrix.rs:391-403"""
        if not (0 <= axis < self.ndim) or not (0 <= index < self.shape[axis]):
            raise IndexError("Index out of bounds")
        shape = self.shape[:axis] + self.shape[axis + 1:]
        stride = self.stride[:axis] + self.stride[axis + 1:]
        return self._view(self.offset + self.stride[axis] * index, shape, stride)

    def slice(self, *slices):
        """slice_dynamic!(...) with python slices (start:stop:step, step > 0); matrix.rs:347-373"""
        if len(slices) > self.ndim:
            raise IndexError("too many slices")
        shape, stride, offset = list(self.shape), list(self.stride), self.offset
        for d, s in enumerate(slices):
            start, stop, step = s.indices(self.shape[d])
            if step <= 0:
                raise ValueError("step must be positive")
            n = max(0, (stop - start + step - 1) // step)
            offset += start * self.stride[d]
            shape[d] = n
            stride[d] = self.stride[d] * step
        return self._view(offset, shape, stride)

    def transpose(self):
        """swap the last two axes (shape_stride.rs:94-114)"""
        if self.ndim < 2:
            raise ValueError("transpose needs at least 2 dims")
        shape, stride = list(self.shape), list(self.stride)
        shape[-1], shape[-2] = shape[-2], shape[-1]
        stride[-1], stride[-2] = stride[-2], stride[-1]
        return self._view(self.offset, shape, stride)

    def transpose_by_index(self, index):
        """shape_stride.rs:137-149"""
        shape = [self.shape[i] for i in index]
        stride = [self.stride[i] for i in index]
        return self._view(self.offset, shape, stride)

    def add_axis(self, axis):
        """shape_stride.rs:186-206"""
        if self.ndim == 0:
            return self._view(self.offset, (1,), (1,))
        shape, stride = [], []
        for i in range(self.ndim):
            if i == axis:
                shape.append(1)
                stride.append(self.stride[i])
            shape.append(self.shape[i])
            stride.append(self.stride[i])
        if axis == self.ndim:
            shape.append(1)
            stride.append(1)
        return self._view(self.offset, shape, stride)

    def reshape(self, new_shape):
        """view with a new shape; the matrix must be default stride (reshape.rs)"""
        new_shape = tuple(new_shape)
        if int(np.prod(new_shape, dtype=np.int64)) != self.num_elm():
            raise ValueError("Number of elements must be the same")
        if not self.is_default_stride_strict():
            raise ValueError("reshape needs a default-stride matrix")
        return self._view(self.offset, new_shape, default_stride(new_shape))

    # ---- copies -------------------------------------------------------------------------
    def copy_from(self, src):
        check(_lib.lib().zenu_hip_copy(_dt(self.dtype), C.byref(self.desc()), C.byref(src.desc()), _stream),
              "copy_from")

    def broadcast(self, source):
        """broadcast.rs:11-43"""
        check(_lib.lib().zenu_hip_broadcast(_dt(self.dtype), C.byref(self.desc()), C.byref(source.desc()), _stream),
              "broadcast")

    def to_default_stride(self):
        out = self.alloc_like()
        out.copy_from(self)
        return out

    def new_matrix(self):
        return self.to_default_stride()

    # ---- binary -------------------------------------------------------------------------
    def _binary_array(self, op, lhs, rhs):
        check(_lib.lib().zenu_hip_binary(op, _dt(self.dtype), C.byref(self.desc()), C.byref(lhs.desc()),
                                         C.byref(rhs.desc()), _stream), "binary")

    def _binary_assign(self, op, rhs):
        check(_lib.lib().zenu_hip_binary_assign(op, _dt(self.dtype), C.byref(self.desc()),
                                                C.byref(rhs.desc()), _stream), "binary_assign")

    def _binary_scalar(self, op, other, scalar):
        check(_lib.lib().zenu_hip_binary_scalar(op, _dt(self.dtype), C.byref(self.desc()),
                                                C.byref(other.desc()), float(scalar), _stream),
              "binary_scalar")

    def _binary_scalar_assign(self, op, scalar):
        check(_lib.lib().zenu_hip_binary_scalar_assign(op, _dt(self.dtype), C.byref(self.desc()),
                                                       float(scalar), _stream), "binary_scalar_assign")

    def _operator(self, op, rhs):
        if isinstance(rhs, Matrix):
            shape = larger_shape(self.shape, rhs.shape)
            out = Matrix.alloc(shape, self.dtype)
            out._binary_array(op, self, rhs)
            return out
        out = self.alloc_like()
        out._binary_scalar(op, self, rhs)
        return out

    def _ioperator(self, op, rhs):
        if isinstance(rhs, Matrix):
            self._binary_assign(op, rhs)
        else:
            self._binary_scalar_assign(op, rhs)
        return self

    def __add__(self, rhs): return self._operator(_lib.ADD, rhs)
    def __sub__(self, rhs): return self._operator(_lib.SUB, rhs)
    def __mul__(self, rhs): return self._operator(_lib.MUL, rhs)
    def __truediv__(self, rhs): return self._operator(_lib.DIV, rhs)
    def __iadd__(self, rhs): return self._ioperator(_lib.ADD, rhs)
    def __isub__(self, rhs): return self._ioperator(_lib.SUB, rhs)
    def __imul__(self, rhs): return self._ioperator(_lib.MUL, rhs)
    def __itruediv__(self, rhs): return self._ioperator(_lib.DIV, rhs)

    # scalar read from device memory (0-d operand): trait methods scalar_ptr / scalar_assign_ptr
    def scalar_ptr(self, op, other, scalar_matrix):
        check(_lib.lib().zenu_hip_binary_scalar_ptr(op, _dt(self.dtype), C.byref(self.desc()),
                                                    C.byref(other.desc()), scalar_matrix.as_ptr(), _stream),
              "binary_scalar_ptr")

    def scalar_assign_ptr(self, op, scalar_matrix):
        check(_lib.lib().zenu_hip_binary_scalar_assign_ptr(op, _dt(self.dtype), C.byref(self.desc()),
                                                           scalar_matrix.as_ptr(), _stream),
              "binary_scalar_assign_ptr")

    # ---- unary --------------------------------------------------------------------------
    def _unary_array(self, fn, other):
        check(_lib.lib().zenu_hip_unary(fn, _dt(self.dtype), C.byref(self.desc()), C.byref(other.desc()),
                                        _stream), "unary")

    def _unary_assign(self, fn):
        check(_lib.lib().zenu_hip_unary_assign(fn, _dt(self.dtype), C.byref(self.desc()), _stream),
              "unary_assign")

    def _unary(self, fn):
        out = self.alloc_like()
        out._unary_array(fn, self)
        return out

    def powf(self, other, scalar):
        check(_lib.lib().zenu_hip_powf(_dt(self.dtype), C.byref(self.desc()), C.byref(other.desc()),
                                       float(scalar), _stream), "powf")

    def powf_array(self, scalar):
        out = self.alloc_like()
        out.powf(self, scalar)
        return out

    def sigmoid(self):
        return self._unary(_lib.SIGMOID)

    def relu(self, other, alpha):
        check(_lib.lib().zenu_hip_relu(_dt(self.dtype), C.byref(self.desc()), C.byref(other.desc()),
                                       float(alpha), _stream), "relu")

    def relu_backward_mask(self, other, alpha):
        check(_lib.lib().zenu_hip_relu_backward_mask(_dt(self.dtype), C.byref(self.desc()),
                                                     C.byref(other.desc()), float(alpha), _stream),
              "relu_backward_mask")

    def tanh_backward(self, gy, x):
        """self = gy / cosh(x)^2: zenu-autograd/src/functions/tanh.rs:30-37 in one pass"""
        check(_lib.lib().zenu_hip_tanh_backward(_dt(self.dtype), C.byref(self.desc()), C.byref(gy.desc()),
                                                C.byref(x.desc()), _stream), "tanh_backward")

    def sigmoid_backward(self, gy, x):
        """self = d sigmoid(x) * gy with the roundings of the autograd chain (activation/sigmoid.rs:7-15)"""
        check(_lib.lib().zenu_hip_sigmoid_backward(_dt(self.dtype), C.byref(self.desc()), C.byref(gy.desc()),
                                                   C.byref(x.desc()), _stream), "sigmoid_backward")

    def relu_backward(self, gy, x, alpha):
        """self = gy * relu_backward_mask(x): zenu-autograd/src/activation/relu.rs:35-44 in one pass"""
        check(_lib.lib().zenu_hip_relu_backward(_dt(self.dtype), C.byref(self.desc()), C.byref(gy.desc()),
                                                C.byref(x.desc()), float(alpha), _stream), "relu_backward")

    def relu_backward_bias_grad(self, gbias, gy, x, alpha):
        """self = gy * relu'(x) and gbias = the column sums of self (the bias gradient of the layer
        before), in one pass over gy"""
        check(_lib.lib().zenu_hip_relu_backward_bias_grad(_dt(self.dtype), C.byref(self.desc()), C.byref(gbias.desc()),
                                                          C.byref(gy.desc()), C.byref(x.desc()), float(alpha), _stream),
              "relu_backward_bias_grad")

    # ---- clip (zenu-matrix/src/operation/clip.rs:289-318) -----------------------------------
    def clip(self, lo, hi):
        out = self.alloc_like()
        check(_lib.lib().zenu_hip_clip(_dt(self.dtype), C.byref(out.desc()), C.byref(self.desc()),
                                       float(lo), float(hi), _stream), "clip")
        return out

    def clip_assign(self, lo, hi):
        check(_lib.lib().zenu_hip_clip(_dt(self.dtype), C.byref(self.desc()), C.byref(self.desc()),
                                       float(lo), float(hi), _stream), "clip_assign")

    def clip_backward_mask(self, lo, hi):
        out = self.alloc_like()
        check(_lib.lib().zenu_hip_clip_backward_mask(_dt(self.dtype), C.byref(out.desc()), C.byref(self.desc()),
                                                     float(lo), float(hi), _stream), "clip_backward_mask")
        return out

    def clip_backward_assign_mask(self, lo, hi):
        check(_lib.lib().zenu_hip_clip_backward_mask(_dt(self.dtype), C.byref(self.desc()), C.byref(self.desc()),
                                                     float(lo), float(hi), _stream), "clip_backward_assign_mask")

    # ---- fused chains -----------------------------------------------------------------------
    def softmax_assign(self, source, axis):
        """softmax.rs:10-25, one launch"""
        if not (0 <= axis < self.ndim):
            raise ZenuHipError(_lib.ERR_AXIS, "softmax_assign", "axis must be less than the number of dimensions")
        check(_lib.lib().zenu_hip_softmax(_dt(self.dtype), C.byref(self.desc()), C.byref(source.desc()),
                                          axis, _stream), "softmax_assign")

    def bias_add_relu(self, z, bias, alpha, pre=None):
        """self = relu(z + bias, alpha); pre (optional) receives z + bias"""
        check(_lib.lib().zenu_hip_bias_add_relu(_dt(self.dtype), C.byref(pre.desc()) if pre is not None else None,
                                                C.byref(self.desc()), C.byref(z.desc()), C.byref(bias.desc()),
                                                float(alpha), _stream), "bias_add_relu")

    # ---- reductions ---------------------------------------------------------------------
    def sum(self, axis, keep_dim=False):
        """sum.rs:9-32"""
        if not (0 <= axis < self.ndim):
            raise ZenuHipError(_lib.ERR_AXIS, "sum", "Invalid axis")
        shape = self.shape[:axis] + self.shape[axis + 1:]
        out = Matrix.alloc(shape, self.dtype)
        check(_lib.lib().zenu_hip_sum_axis(_dt(self.dtype), C.byref(out.desc()), C.byref(self.desc()),
                                           axis, _stream), "sum_axis")
        return out.add_axis(axis) if keep_dim else out

    def sum_all(self):
        out = Matrix.alloc((), self.dtype)
        check(_lib.lib().zenu_hip_sum_all(_dt(self.dtype), out.as_ptr(), C.byref(self.desc()), _stream),
              "sum_all")
        return out

    def max_idx(self):
        """max.rs:45-56: N-d index of the first maximum"""
        if self.ndim == 0:
            return ()
        idx = Matrix.alloc((), np.int64)
        check(_lib.lib().zenu_hip_max_idx(_dt(self.dtype), idx.as_ptr(), None, C.byref(self.desc()), _stream),
              "max_idx")
        flat = int(idx.to_numpy())
        return tuple(int(i) for i in np.unravel_index(flat, self.shape))

    def max_item(self):
        val = Matrix.alloc((), self.dtype)
        idx = Matrix.alloc((), np.int64)
        check(_lib.lib().zenu_hip_max_idx(_dt(self.dtype), idx.as_ptr(), val.as_ptr(), C.byref(self.desc()),
                                          _stream), "max_item")
        return val.to_numpy()[()]

    def max_axis(self, axis, keep_dim=False):
        """max.rs:67-99"""
        if not (0 <= axis < self.ndim):
            raise ZenuHipError(_lib.ERR_AXIS, "max_axis", "max_axis: Axis out of bounds")
        shape = self.shape[:axis] + self.shape[axis + 1:]
        out = Matrix.alloc(shape, self.dtype)
        check(_lib.lib().zenu_hip_max_axis(_dt(self.dtype), C.byref(out.desc()), C.byref(self.desc()),
                                           axis, _stream), "max_axis")
        return out.add_axis(axis) if keep_dim else out

    def max_axis_idx_ravel(self, axis):
        """max.rs:103-134"""
        if not (0 <= axis < self.ndim):
            raise ZenuHipError(_lib.ERR_AXIS, "max_axis_idx_ravel", "max_axis: Axis out of bounds")
        shape = self.shape[:axis] + self.shape[axis + 1:]
        out = Matrix.alloc(shape, np.int64)
        check(_lib.lib().zenu_hip_max_axis_idx(_dt(self.dtype), out.as_ptr(), C.byref(self.desc()), axis,
                                               _stream), "max_axis_idx")
        return [int(i) for i in out.to_numpy().reshape(-1)]

    def asum(self):
        out = Matrix.alloc((), self.dtype)
        check(_lib.lib().zenu_hip_asum(_dt(self.dtype), out.as_ptr(), C.byref(self.desc()), _stream), "asum")
        return out.to_numpy()[()]

    def mean(self, axis=None, keep_dim=False):
        """mean.rs:9-20: sum(axis) / n; without an axis asum() / num_elm -- the mean of |x|, as the
        reference computes it -- returned as a 0-d matrix"""
        if axis is not None:
            return self.sum(axis, keep_dim) / self.dtype.type(self.shape[axis])
        n = 1
        for d in self.shape:
            n *= d
        return Matrix.from_numpy(np.asarray(self.asum() / self.dtype.type(n), dtype=self.dtype))

    def variance(self, axis=None, keep_dim=False):
        """var.rs:19-26: mean((x - mean(x, keep))^2), each step an operator of its own"""
        diff = self - self.mean(axis, True)
        return (diff * diff).mean(axis, keep_dim)

    def index_item(self, index):
        return self.to_numpy()[tuple(index)]


def _make_named(name, op):
    def array(self, lhs, rhs): self._binary_array(op, lhs, rhs)
    def assign(self, rhs): self._binary_assign(op, rhs)
    def scalar(self, other, s): self._binary_scalar(op, other, s)
    def scalar_assign(self, s): self._binary_scalar_assign(op, s)
    setattr(Matrix, f"{name}_array", array)
    setattr(Matrix, f"{name}_assign", assign)
    setattr(Matrix, f"{name}_scalar", scalar)
    setattr(Matrix, f"{name}_scalar_assign", scalar_assign)


for _n, _o in (("add", _lib.ADD), ("sub", _lib.SUB), ("mul", _lib.MUL), ("div", _lib.DIV)):
    _make_named(_n, _o)


def _make_unary(name, fn):
    def out(self): return self._unary(fn)
    def array(self, other): self._unary_array(fn, other)
    def assign(self): self._unary_assign(fn)
    setattr(Matrix, name, out)
    setattr(Matrix, f"{name}_array", array)
    setattr(Matrix, f"{name}_assign", assign)


for _n, _f in (("exp", _lib.EXP), ("log", _lib.LOG), ("tanh", _lib.TANH), ("sqrt", _lib.SQRT),
               ("abs", _lib.ABS), ("sin", _lib.SIN), ("cos", _lib.COS), ("tan", _lib.TAN),
               ("asin", _lib.ASIN), ("acos", _lib.ACOS), ("atan", _lib.ATAN), ("sinh", _lib.SINH),
               ("cosh", _lib.COSH),
               # not in the reference: f32 tanh within 2 ulp of `tanh` on every argument, memory-bound
               ("tanh_ulp2", _lib.TANH_ULP2)):
    _make_unary(_n, _f)


def larger_shape(x, y):
    """Result shape an operator allocates (impl_ops.rs:69-76, dim_dyn.rs:24-58)."""
    x, y = tuple(x), tuple(y)

    def is_include(s, o):
        if len(s) < len(o):
            return is_include(o, s)
        return all(s[len(s) - 1 - i] == o[len(o) - 1 - i] for i in range(len(o)))

    def is_include_broadcast(s, o):
        return all(s[len(s) - 1 - i] == o[len(o) - 1 - i] or o[len(o) - 1 - i] == 1 for i in range(len(o)))

    if len(x) > len(y):
        return x
    if len(x) < len(y):
        return y
    if is_include_broadcast(x, y):
        return x
    if is_include_broadcast(y, x):
        return y
    raise ZenuHipError(_lib.ERR_SHAPE, "larger_shape", "This is bug please make issue")


def softmax_backward(y, gy, axis):
    """gx = y*gy - y*sum(y*gy, axis) (zenu-autograd/src/loss/softmax.rs:33-40), one launch"""
    gx = y.alloc_like()
    check(_lib.lib().zenu_hip_softmax_backward(_dt(y.dtype), C.byref(gx.desc()), C.byref(y.desc()),
                                               C.byref(gy.desc()), axis, _stream), "softmax_backward")
    return gx


def cross_entropy(pred, ans):
    """(loss, prob) of zenu-autograd/src/loss/cross_entropy.rs:12-23 for pred, ans [N, C]"""
    loss = Matrix.alloc((), pred.dtype)
    prob = pred.alloc_like()
    check(_lib.lib().zenu_hip_softmax_cross_entropy(_dt(pred.dtype), C.byref(loss.desc()), C.byref(prob.desc()),
                                                    C.byref(pred.desc()), C.byref(ans.desc()), _stream),
          "cross_entropy")
    return loss, prob


def cross_entropy_backward(prob, ans, gloss=None):
    """d loss / d pred from the softmax output kept by cross_entropy()"""
    gpred = prob.alloc_like()
    check(_lib.lib().zenu_hip_softmax_cross_entropy_backward(
        _dt(prob.dtype), C.byref(gpred.desc()), C.byref(prob.desc()), C.byref(ans.desc()),
        C.byref(gloss.desc()) if gloss is not None else None, _stream), "cross_entropy_backward")
    return gpred


def cross_entropy_backward_bias_grad(prob, ans, gbias, gloss=None):
    """cross_entropy_backward() that also writes the column sums of the gradient to gbias"""
    gpred = prob.alloc_like()
    check(_lib.lib().zenu_hip_softmax_cross_entropy_backward_bias_grad(
        _dt(prob.dtype), C.byref(gpred.desc()), C.byref(gbias.desc()), C.byref(prob.desc()), C.byref(ans.desc()),
        C.byref(gloss.desc()) if gloss is not None else None, _stream), "cross_entropy_backward_bias_grad")
    return gpred


def conv2d_bias_add(input, bias, output):
    """zenu-matrix/src/nn/conv/mod.rs:84-95: output[N,C,H,W] = input + bias[1,C,1,1], one launch"""
    if tuple(input.shape) != tuple(output.shape):
        raise ZenuHipError(_lib.ERR_SHAPE, "conv2d_bias_add", "input and output shapes differ")
    if bias.ndim != 4 or input.ndim != 4 or (bias.shape[0], bias.shape[2], bias.shape[3]) != (1, 1, 1) \
            or bias.shape[1] != output.shape[1]:
        raise ZenuHipError(_lib.ERR_SHAPE, "conv2d_bias_add", "bias must be [1, C, 1, 1]")
    output.add_array(input, bias)


def conv2d_bias_bkwd(d_output, d_bias):
    """zenu-matrix/src/nn/conv/mod.rs:98-107 with the CPU device's definition (cpu/bias.rs:18-25):
    d_bias[1,C,1,1] = d_output[N,C,H,W] summed over axes 0, 2 and 3, in that order"""
    if d_bias.ndim != 4 or d_output.ndim != 4 or (d_bias.shape[0], d_bias.shape[2], d_bias.shape[3]) != (1, 1, 1) \
            or d_bias.shape[1] != d_output.shape[1]:
        raise ZenuHipError(_lib.ERR_SHAPE, "conv2d_bias_bkwd", "d_bias must be [1, C, 1, 1]")
    sum_to(d_output, d_bias)


def _axis_range(m, axis, start, stop):
    return m.slice(*([slice(None)] * axis + [slice(start, stop)]))


def stack(matrices, axis):
    """zenu-matrix/src/operation/stack.rs:18-58: the inputs laid one after the other along `axis`
    (the output's extent there is len(matrices) times the inputs'); one strided copy per input
    where the reference copies index by index"""
    if not matrices:
        raise ZenuHipError(_lib.ERR_ARG, "stack", "No matrices to stack")
    first = tuple(matrices[0].shape)
    if any(tuple(m.shape) != first for m in matrices):
        raise ZenuHipError(_lib.ERR_SHAPE, "stack", "All matrices must have the same shape")
    if not (0 <= axis < len(first)):      # the reference admits axis == ndim and then indexes out of bounds
        raise ZenuHipError(_lib.ERR_AXIS, "stack", "Axis out of bounds for stack")
    n = first[axis]
    shape = list(first)
    shape[axis] = n * len(matrices)
    out = Matrix.alloc(shape, matrices[0].dtype)
    for i, m in enumerate(matrices):
        _axis_range(out, axis, i * n, (i + 1) * n).copy_from(m)
    return out


def split(matrix, axis, num_splits):
    """zenu-matrix/src/operation/split.rs:20-58: num_splits equal pieces along `axis`, each a new
    matrix; one strided copy per piece"""
    if not (0 <= axis < matrix.ndim):
        raise ZenuHipError(_lib.ERR_AXIS, "split", "Axis out of bounds")
    if num_splits <= 0 or matrix.shape[axis] % num_splits:
        raise ZenuHipError(_lib.ERR_SHAPE, "split", "Size along axis is not divisible by num_splits")
    n = matrix.shape[axis] // num_splits
    shape = list(matrix.shape)
    shape[axis] = n
    outs = []
    for i in range(num_splits):
        o = Matrix.alloc(shape, matrix.dtype)
        o.copy_from(_axis_range(matrix, axis, i * n, (i + 1) * n))
        outs.append(o)
    return outs


def sum_to(source, target):
    """sum.rs:35-94: reduce `source` into the (smaller) `target` in place"""
    check(_lib.lib().zenu_hip_sum_to(_dt(source.dtype), C.byref(target.desc()), C.byref(source.desc()),
                                     _stream), "sum_to")
