"""numpy-facing wrapper of the CPU oracle (oracle/libzenu_oracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the cpu_baseline leg of
bench.py.  The product (zenu_amd, libzenu_hip.so) never imports or links it.

Arrays are passed as strided views: any numpy view (sliced, transposed, broadcast_to) maps to a
zo_view with element strides, which is what ZeNu's Matrix views are.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libzenu_oracle.so")

ADD, SUB, MUL, DIV = 0, 1, 2, 3
(EXP, LOG, TANH, SQRT, ABS, SIN, COS, TAN, ASIN, ACOS, ATAN, SINH, COSH) = range(13)


class View(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("ndim", C.c_int32), ("reserved", C.c_int32),
                ("shape", C.c_int64 * 6), ("stride", C.c_int64 * 6)]


class OracleError(RuntimeError):
    """The reference would panic here (rank / shape / axis)."""

    def __init__(self, code, where):
        self.code = code
        super().__init__(f"{where}: oracle status {code}")


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "libzenu_oracle.so"], stdout=subprocess.DEVNULL)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.zo_leaf_calls.restype = C.c_uint64
        for s, ct in (("f32", C.c_float), ("f64", C.c_double)):
            getattr(_lib, f"zo_asum_{s}").restype = ct
            getattr(_lib, f"zo_asum_leaf_{s}").restype = ct
            getattr(_lib, f"zo_max_idx_leaf_{s}").restype = C.c_size_t
    return _lib


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32", C.c_float
    if dtype == np.float64:
        return "f64", C.c_double
    raise TypeError(dtype)


def view(a):
    v = View()
    v.ptr = a.ctypes.data
    v.ndim = a.ndim
    for i in range(a.ndim):
        v.shape[i] = a.shape[i]
        assert a.strides[i] % a.itemsize == 0 and a.strides[i] >= 0
        v.stride[i] = a.strides[i] // a.itemsize
    return v


def _chk(rc, where):
    if rc != 0:
        raise OracleError(rc, where)


def leaf_calls():
    return int(lib().zo_leaf_calls())


def reset_leaf_calls():
    lib().zo_reset_leaf_calls()


# ---- Matrix-level ops: all write into `to` (a writable numpy view) -------------------------------

def binary_array(op, to, lhs, rhs):
    s, _ = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_binary_array_{s}")(op, C.byref(view(to)), C.byref(view(lhs)), C.byref(view(rhs))),
         "binary_array")


def binary_assign(op, to, rhs):
    s, _ = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_binary_assign_{s}")(op, C.byref(view(to)), C.byref(view(rhs))), "binary_assign")


def binary_scalar(op, to, other, scalar):
    s, ct = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_binary_scalar_{s}")(op, C.byref(view(to)), C.byref(view(other)), ct(scalar)),
         "binary_scalar")


def binary_scalar_assign(op, to, scalar):
    s, ct = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_binary_scalar_assign_{s}")(op, C.byref(view(to)), ct(scalar)),
         "binary_scalar_assign")


def unary(fn, to, other):
    s, _ = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_unary_{s}")(fn, C.byref(view(to)), C.byref(view(other))), "unary")


def unary_assign(fn, to):
    s, _ = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_unary_assign_{s}")(fn, C.byref(view(to))), "unary_assign")


def powf(to, other, scalar):
    s, ct = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_powf_{s}")(C.byref(view(to)), C.byref(view(other)), ct(scalar)), "powf")


def relu(to, other, alpha):
    s, ct = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_relu_{s}")(C.byref(view(to)), C.byref(view(other)), ct(alpha)), "relu")


def clip(to, other, lo, hi):
    s, ct = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_clip_{s}")(C.byref(view(to)), C.byref(view(other)), ct(lo), ct(hi)), "clip")


def clip_backward_mask(mask, other, lo, hi):
    s, ct = _sfx(mask.dtype)
    _chk(getattr(lib(), f"zo_clip_backward_mask_{s}")(C.byref(view(mask)), C.byref(view(other)), ct(lo), ct(hi)),
         "clip_backward_mask")


def relu_backward_mask(to, other, alpha):
    s, ct = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_relu_backward_mask_{s}")(C.byref(view(to)), C.byref(view(other)), ct(alpha)),
         "relu_backward_mask")


def sigmoid(to, x):
    s, _ = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_sigmoid_{s}")(C.byref(view(to)), C.byref(view(x))), "sigmoid")


SIGMOID_COMPOSITE = 13


def unary_range_hash(fn, first, count, block_log2, nthreads=1):
    """one 64-bit sum per block of 2^block_log2 f32 bit patterns of [first, first + count): every
    pattern through unary function `fn` (or SIGMOID_COMPOSITE), argument and result bits hashed and added"""
    sums = np.zeros(count >> block_log2, dtype=np.uint64)
    f = lib().zo_unary_range_hash_f32
    f.argtypes = [C.c_int, C.c_uint64, C.c_uint64, C.c_int, C.c_void_p, C.c_int]
    f.restype = C.c_int
    _chk(f(fn, first, count, block_log2, sums.ctypes.data, nthreads), "unary_range_hash")
    return sums


def powf_range_hash(exponent, first, count, block_log2, nthreads=1):
    sums = np.zeros(count >> block_log2, dtype=np.uint64)
    f = lib().zo_powf_range_hash_f32
    f.argtypes = [C.c_float, C.c_uint64, C.c_uint64, C.c_int, C.c_void_p, C.c_int]
    f.restype = C.c_int
    _chk(f(exponent, first, count, block_log2, sums.ctypes.data, nthreads), "powf_range_hash")
    return sums


def unary_range_hash_f64(fn, first, count, block_log2, step, offset, salt, nthreads=1):
    """f64: argument number i has the high word i * step + offset and a pseudo-random low word (range_arg_f64)"""
    sums = np.zeros(count >> block_log2, dtype=np.uint64)
    f = lib().zo_unary_range_hash_f64
    f.argtypes = [C.c_int, C.c_uint64, C.c_uint64, C.c_int, C.c_uint32, C.c_uint32, C.c_uint64, C.c_void_p, C.c_int]
    f.restype = C.c_int
    _chk(f(fn, first, count, block_log2, step, offset, salt, sums.ctypes.data, nthreads), "unary_range_hash_f64")
    return sums


def powf_range_hash_f64(exponent, first, count, block_log2, step, offset, salt, nthreads=1):
    """the same for pow(x, exponent) over the sampled f64 bases"""
    sums = np.zeros(count >> block_log2, dtype=np.uint64)
    f = lib().zo_powf_range_hash_f64
    f.argtypes = [C.c_double, C.c_uint64, C.c_uint64, C.c_int, C.c_uint32, C.c_uint32, C.c_uint64, C.c_void_p, C.c_int]
    f.restype = C.c_int
    _chk(f(exponent, first, count, block_log2, step, offset, salt, sums.ctypes.data, nthreads), "powf_range_hash_f64")
    return sums


def range_arg_f64(i, step, offset, salt):
    f = lib().zo_range_arg_f64
    f.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint64]
    f.restype = C.c_uint64
    return int(f(i, step, offset, salt))


def range_hash_term(arg_bits, res_bits):
    f = lib().zo_range_hash_term
    f.argtypes = [C.c_uint32, C.c_uint32]
    f.restype = C.c_uint64
    return int(f(arg_bits, res_bits))


def copy_from(to, src):
    s, _ = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_copy_from_{s}")(C.byref(view(to)), C.byref(view(src))), "copy_from")


def broadcast(to, source):
    s, _ = _sfx(to.dtype)
    _chk(getattr(lib(), f"zo_broadcast_{s}")(C.byref(view(to)), C.byref(view(source))), "broadcast")


def sum_axis(src, axis, keep_dim=False):
    s, _ = _sfx(src.dtype)
    if not (0 <= axis < src.ndim):
        raise OracleError(3, "sum")
    shape = src.shape[:axis] + src.shape[axis + 1:]
    out = np.empty(shape, dtype=src.dtype)
    _chk(getattr(lib(), f"zo_sum_{s}")(C.byref(view(src)), axis, C.c_void_p(out.ctypes.data)), "sum")
    return np.expand_dims(out, axis) if keep_dim else out


def sum_to(src, target):
    s, _ = _sfx(src.dtype)
    _chk(getattr(lib(), f"zo_sum_to_{s}")(C.byref(view(src)), C.byref(view(target))), "sum_to")


def max_idx(src):
    s, _ = _sfx(src.dtype)
    idx = (C.c_int64 * 6)()
    _chk(getattr(lib(), f"zo_max_idx_{s}")(C.byref(view(src)), idx), "max_idx")
    return tuple(int(idx[i]) for i in range(src.ndim))


def max_item(src):
    s, ct = _sfx(src.dtype)
    out = ct()
    _chk(getattr(lib(), f"zo_max_item_{s}")(C.byref(view(src)), C.byref(out)), "max_item")
    return np.dtype(src.dtype).type(out.value)


def max_axis(src, axis, keep_dim=False):
    s, _ = _sfx(src.dtype)
    if not (0 <= axis < src.ndim):
        raise OracleError(3, "max_axis")
    shape = src.shape[:axis] + src.shape[axis + 1:]
    out = np.empty(shape, dtype=src.dtype)
    _chk(getattr(lib(), f"zo_max_axis_{s}")(C.byref(view(src)), axis, C.c_void_p(out.ctypes.data)), "max_axis")
    return np.expand_dims(out, axis) if keep_dim else out


def max_axis_idx_ravel(src, axis):
    s, _ = _sfx(src.dtype)
    if not (0 <= axis < src.ndim):
        raise OracleError(3, "max_axis_idx_ravel")
    n = int(np.prod(src.shape[:axis] + src.shape[axis + 1:], dtype=np.int64))
    out = np.empty(n, dtype=np.int64)
    _chk(getattr(lib(), f"zo_max_axis_idx_ravel_{s}")(C.byref(view(src)), axis, C.c_void_p(out.ctypes.data)),
         "max_axis_idx_ravel")
    return out


def asum(src):
    s, _ = _sfx(src.dtype)
    return np.dtype(src.dtype).type(getattr(lib(), f"zo_asum_{s}")(C.byref(view(src))))


# ---- optimizers on flat contiguous arrays (updated in place) ---------------------------------------

def _flatptr(a):
    assert a.flags["C_CONTIGUOUS"]
    return C.c_void_p(a.ctypes.data)


def sgd_update(p, g, lr):
    s, ct = _sfx(p.dtype)
    getattr(lib(), f"zo_sgd_update_{s}")(_flatptr(p), _flatptr(g), C.c_size_t(p.size), ct(lr))


def adam_update(p, g, m, v, lr, beta1, beta2, eps, step):
    s, ct = _sfx(p.dtype)
    getattr(lib(), f"zo_adam_update_{s}")(_flatptr(p), _flatptr(g), _flatptr(m), _flatptr(v),
                                         C.c_size_t(p.size), ct(lr), ct(beta1), ct(beta2), ct(eps), ct(step))


def adamw_update(p, g, m, v, lr, beta1, beta2, eps, weight_decay, is_weight, step):
    s, ct = _sfx(p.dtype)
    getattr(lib(), f"zo_adamw_update_{s}")(_flatptr(p), _flatptr(g), _flatptr(m), _flatptr(v),
                                          C.c_size_t(p.size), ct(lr), ct(beta1), ct(beta2), ct(eps),
                                          ct(weight_decay), C.c_int(1 if is_weight else 0), ct(step))


def adam_update_fused(p, g, m, v, lr, beta1, beta2, eps, weight_decay, is_weight, adamw, step):
    s, ct = _sfx(p.dtype)
    getattr(lib(), f"zo_adam_update_fused_{s}")(_flatptr(p), _flatptr(g), _flatptr(m), _flatptr(v),
                                               C.c_size_t(p.size), ct(lr), ct(beta1), ct(beta2), ct(eps),
                                               ct(weight_decay), C.c_int(1 if is_weight else 0),
                                               C.c_int(1 if adamw else 0), ct(step))
