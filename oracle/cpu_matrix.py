"""CpuMatrix: the oracle behind the same method names as zenu_amd.Matrix.

This is the `Cpu` leg of the reference's run_mat_test! pattern (zenu-test/src/lib.rs:62-91): one
generic test body, instantiated once with the CPU oracle and once with the HIP device.
"""
import numpy as np

import zenu_oracle as zo


class CpuMatrix:
    Error = zo.OracleError

    def __init__(self, arr):
        self.a = arr  # a numpy view; strides carry the Matrix view

    # constructors
    @staticmethod
    def alloc(shape, dtype=np.float32):
        return CpuMatrix(np.empty(tuple(shape), dtype=dtype))

    @staticmethod
    def zeros(shape, dtype=np.float32):
        return CpuMatrix(np.zeros(tuple(shape), dtype=dtype))

    @staticmethod
    def from_numpy(arr):
        return CpuMatrix(np.array(arr, copy=True, order="C"))

    @staticmethod
    def from_vec(vec, shape, dtype=np.float32):
        return CpuMatrix(np.asarray(vec, dtype=dtype).reshape(tuple(shape)).copy())

    def alloc_like(self):
        return CpuMatrix.alloc(self.a.shape, self.a.dtype)

    @property
    def shape(self):
        return tuple(self.a.shape)

    @property
    def dtype(self):
        return self.a.dtype

    @property
    def ndim(self):
        return self.a.ndim

    def to_numpy(self):
        return np.array(self.a, copy=True, order="C")

    def index_item(self, index):
        return self.a[tuple(index)]

    # views
    def index_axis(self, axis, index):
        # a view also when the result is 0-d (plain integer indexing would return a numpy scalar)
        return CpuMatrix(np.squeeze(self.a[(slice(None),) * axis + (slice(index, index + 1),)], axis=axis))

    def slice(self, *slices):
        return CpuMatrix(self.a[tuple(slices)])

    def transpose(self):
        return CpuMatrix(np.swapaxes(self.a, -1, -2))

    def transpose_by_index(self, index):
        return CpuMatrix(np.transpose(self.a, index))

    def add_axis(self, axis):
        return CpuMatrix(np.expand_dims(self.a, axis))

    def reshape(self, new_shape):
        assert self.a.flags["C_CONTIGUOUS"]
        return CpuMatrix(self.a.reshape(tuple(new_shape)))

    # copies
    def copy_from(self, src):
        zo.copy_from(self.a, src.a)

    def broadcast(self, source): zo.broadcast(self.a, source.a)

    def to_default_stride(self):
        out = self.alloc_like()
        out.copy_from(self)
        return out

    # operators (impl_ops.rs)
    def _operator(self, op, rhs):
        if isinstance(rhs, CpuMatrix):
            from zenu_amd.matrix import larger_shape  # pure shape arithmetic, no device call
            out = CpuMatrix.alloc(larger_shape(self.shape, rhs.shape), self.dtype)
            zo.binary_array(op, out.a, self.a, rhs.a)
            return out
        out = self.alloc_like()
        zo.binary_scalar(op, out.a, self.a, rhs)
        return out

    def _ioperator(self, op, rhs):
        if isinstance(rhs, CpuMatrix):
            zo.binary_assign(op, self.a, rhs.a)
        else:
            zo.binary_scalar_assign(op, self.a, rhs)
        return self

    def __add__(self, r): return self._operator(zo.ADD, r)
    def __sub__(self, r): return self._operator(zo.SUB, r)
    def __mul__(self, r): return self._operator(zo.MUL, r)
    def __truediv__(self, r): return self._operator(zo.DIV, r)
    def __iadd__(self, r): return self._ioperator(zo.ADD, r)
    def __isub__(self, r): return self._ioperator(zo.SUB, r)
    def __imul__(self, r): return self._ioperator(zo.MUL, r)
    def __itruediv__(self, r): return self._ioperator(zo.DIV, r)

    def powf(self, other, scalar): zo.powf(self.a, other.a, scalar)

    def powf_array(self, scalar):
        out = self.alloc_like()
        out.powf(self, scalar)
        return out

    def sigmoid(self):
        out = self.alloc_like()
        zo.sigmoid(out.a, self.a)
        return out

    def relu(self, other, alpha): zo.relu(self.a, other.a, alpha)
    def relu_backward_mask(self, other, alpha): zo.relu_backward_mask(self.a, other.a, alpha)

    def tanh_backward(self, gy, x):
        """zenu-autograd/src/functions/tanh.rs:30-37: cosh(x), cosh * cosh, gy / that"""
        c = x.cosh()
        self.div_array(gy, c * c)

    def sigmoid_backward(self, gy, x):
        """backward of activation/sigmoid.rs:7-15, node by node: add passes gy on; mul(half, th) gives
        half * gy (functions/mul.rs:35-44); tanh divides by cosh(x * half)^2; mul(x, half) gives g * half"""
        half = CpuMatrix.from_vec([0.5], (), self.dtype)
        g1 = half * gy
        c = (x * half).cosh()
        g2 = g1 / (c * c)
        self.mul_array(g2, half)

    def relu_backward(self, gy, x, alpha):
        """zenu-autograd/src/activation/relu.rs:35-44: mask, then gy * mask"""
        mask = x.alloc_like()
        mask.relu_backward_mask(x, alpha)
        self.mul_array(gy, mask)

    def relu_backward_bias_grad(self, gbias, gy, x, alpha):
        """the two nodes the fused call stands for: relu backward, then the bias gradient's sum_to
        (zenu-autograd/src/lib.rs:466-486)"""
        self.relu_backward(gy, x, alpha)
        sum_to(self, gbias)

    # clip.rs:289-318
    def clip(self, lo, hi):
        out = self.alloc_like()
        zo.clip(out.a, self.a, lo, hi)
        return out

    def clip_assign(self, lo, hi): zo.clip(self.a, self.a, lo, hi)

    def clip_backward_mask(self, lo, hi):
        out = self.alloc_like()
        zo.clip_backward_mask(out.a, self.a, lo, hi)
        return out

    def clip_backward_assign_mask(self, lo, hi): zo.clip_backward_mask(self.a, self.a, lo, hi)

    def softmax_assign(self, source, axis):
        """softmax.rs:10-25, op by op"""
        if not (0 <= axis < self.ndim):
            raise zo.OracleError("axis must be less than the number of dimensions")
        max_diff = source - source.max_axis(axis, True)
        output = max_diff.exp()
        total = output.sum(axis, True)
        output /= total
        self.copy_from(output)

    def bias_add_relu(self, z, bias, alpha, pre=None):
        """Linear::call's `+ bias` (linear.rs:27-31) followed by relu (activation/relu.rs:24-33)"""
        a = z + bias
        if pre is not None:
            pre.copy_from(a)
        self.relu(a, alpha)

    # reductions
    def sum(self, axis, keep_dim=False): return CpuMatrix(zo.sum_axis(self.a, axis, keep_dim))

    def sum_all(self):
        out = CpuMatrix.zeros((), self.dtype)
        zo.sum_to(self.a, out.a)
        return out

    def max_idx(self): return zo.max_idx(self.a)
    def max_item(self): return zo.max_item(self.a)
    def max_axis(self, axis, keep_dim=False): return CpuMatrix(zo.max_axis(self.a, axis, keep_dim))
    def max_axis_idx_ravel(self, axis): return [int(i) for i in zo.max_axis_idx_ravel(self.a, axis)]
    def asum(self): return zo.asum(self.a)

    def mean(self, axis=None, keep_dim=False):
        """mean.rs:9-20"""
        if axis is not None:
            return self.sum(axis, keep_dim) / self.dtype.type(self.shape[axis])
        n = 1
        for d in self.shape:
            n *= d
        return CpuMatrix.from_numpy(np.asarray(self.asum() / self.dtype.type(n), dtype=self.dtype))

    def variance(self, axis=None, keep_dim=False):
        """var.rs:19-26"""
        diff = self - self.mean(axis, True)
        return (diff * diff).mean(axis, keep_dim)


def _named(name, op):
    setattr(CpuMatrix, f"{name}_array", lambda self, l, r: zo.binary_array(op, self.a, l.a, r.a))
    setattr(CpuMatrix, f"{name}_assign", lambda self, r: zo.binary_assign(op, self.a, r.a))
    setattr(CpuMatrix, f"{name}_scalar", lambda self, o, s: zo.binary_scalar(op, self.a, o.a, s))
    setattr(CpuMatrix, f"{name}_scalar_assign", lambda self, s: zo.binary_scalar_assign(op, self.a, s))


for _n, _o in (("add", zo.ADD), ("sub", zo.SUB), ("mul", zo.MUL), ("div", zo.DIV)):
    _named(_n, _o)


def _unary(name, fn):
    def out(self):
        r = self.alloc_like()
        zo.unary(fn, r.a, self.a)
        return r
    setattr(CpuMatrix, name, out)
    setattr(CpuMatrix, f"{name}_array", lambda self, o: zo.unary(fn, self.a, o.a))
    setattr(CpuMatrix, f"{name}_assign", lambda self: zo.unary_assign(fn, self.a))


for _n, _f in (("exp", zo.EXP), ("log", zo.LOG), ("tanh", zo.TANH), ("sqrt", zo.SQRT), ("abs", zo.ABS),
               ("sin", zo.SIN), ("cos", zo.COS), ("tan", zo.TAN), ("asin", zo.ASIN), ("acos", zo.ACOS),
               ("atan", zo.ATAN), ("sinh", zo.SINH), ("cosh", zo.COSH)):
    _unary(_n, _f)


def stack(matrices, axis):
    """zenu-matrix/src/operation/stack.rs:18-58, index by index as the reference copies"""
    first = tuple(matrices[0].shape)
    assert all(tuple(m.shape) == first for m in matrices), "All matrices must have the same shape"
    n = first[axis]
    shape = list(first)
    shape[axis] = n * len(matrices)
    out = CpuMatrix.alloc(shape, matrices[0].dtype)
    for i, m in enumerate(matrices):
        for j in range(n):
            out.index_axis(axis, i * n + j).copy_from(m.index_axis(axis, j))
    return out


def split(matrix, axis, num_splits):
    """zenu-matrix/src/operation/split.rs:20-58"""
    assert matrix.shape[axis] % num_splits == 0
    n = matrix.shape[axis] // num_splits
    shape = list(matrix.shape)
    shape[axis] = n
    outs = []
    for i in range(num_splits):
        o = CpuMatrix.alloc(shape, matrix.dtype)
        for j in range(n):
            o.index_axis(axis, j).copy_from(matrix.index_axis(axis, i * n + j))
        outs.append(o)
    return outs


def sum_to(source, target):
    zo.sum_to(source.a, target.a)


def conv2d_bias_add(input, bias, output):
    """ConvBias for Cpu, zenu-matrix/src/nn/conv/cpu/bias.rs:10-16"""
    output.add_array(input, bias)


def conv2d_bias_bkwd(d_output, d_bias):
    """zenu-matrix/src/nn/conv/cpu/bias.rs:18-25: sum(0, true), sum(2, true), sum(3, true), copy_from"""
    d_bias.copy_from(d_output.sum(0, True).sum(2, True).sum(3, True))


def softmax_backward(y, gy, axis):
    """SoftMax::backward, zenu-autograd/src/loss/softmax.rs:33-40"""
    gx = y * gy
    sum_gx = gx.sum(axis, True)
    return gx - (y * sum_gx)


def cross_entropy(pred, ans):
    """zenu-autograd/src/loss/cross_entropy.rs:12-23 -> (loss, softmax output)"""
    prob = pred.alloc_like()
    prob.softmax_assign(pred, 1)
    y_log_pred = ans * prob.log()
    total = CpuMatrix.zeros((), pred.dtype)
    sum_to(y_log_pred, total)
    neg_n = CpuMatrix.from_vec([-float(pred.shape[0])], (), pred.dtype)
    return total / neg_n, prob


def cross_entropy_backward_bias_grad(prob, ans, gbias, gloss=None):
    """cross_entropy_backward, then the bias gradient's sum_to"""
    g = cross_entropy_backward(prob, ans, gloss)
    sum_to(g, gbias)
    return g


def cross_entropy_backward(prob, ans, gloss=None):
    """backward of div (x side), sum_to (broadcast), mul (log side), log, softmax, in that order
    (functions/div.rs, sum_to.rs, mul.rs, log.rs, loss/softmax.rs:33-40)"""
    dt = prob.dtype
    if gloss is None:
        gloss = CpuMatrix.from_vec([1.0], (), dt)
    neg_n = CpuMatrix.from_vec([-float(prob.shape[0])], (), dt)
    g_total = gloss / neg_n
    g_yl = CpuMatrix.zeros(prob.shape, dt)
    g_yl += g_total
    g_log = ans * g_yl
    g_prob = g_log / prob
    return softmax_backward(prob, g_prob, 1)
