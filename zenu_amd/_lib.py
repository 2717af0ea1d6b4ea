"""ctypes binding of libzenu_hip.so (the C ABI declared in include/zenu_hip.h).

The library is built in-tree by zenu_amd/csrc/Makefile.  There is no CPU fallback: if the
shared object is missing, loading fails loudly.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libzenu_hip.so")

MAX_DIM = 6
F32, F64 = 0, 1
ADD, SUB, MUL, DIV = 0, 1, 2, 3
(EXP, LOG, TANH, SQRT, ABS, SIN, COS, TAN, ASIN, ACOS, ATAN, SINH, COSH, SIGMOID, TANH_ULP2) = range(15)

(OK, ERR_RANK, ERR_SHAPE, ERR_AXIS, ERR_ARG, ERR_HIP, ERR_OOM, ERR_UNSUPPORTED, ERR_NOT_OWNED, ERR_NOT_INIT,
 ERR_SCRATCH_LIMIT) = range(11)


class Tensor(C.Structure):
    """zenu_tensor_t"""
    _fields_ = [("ptr", C.c_void_p), ("ndim", C.c_int32), ("reserved", C.c_int32),
                ("shape", C.c_int64 * MAX_DIM), ("stride", C.c_int64 * MAX_DIM)]


class MempoolStats(C.Structure):
    """zenu_mempool_stats_t"""
    _fields_ = [(n, C.c_uint64) for n in (
        "bytes_in_use", "bytes_cached", "bytes_reserved", "n_alloc_calls", "n_cache_hits",
        "n_driver_allocs", "n_driver_frees", "n_oom_retries")]


class ZenuHipError(RuntimeError):
    def __init__(self, status, where, detail=""):
        self.status = status
        super().__init__(f"{where}: status {status} ({detail})")


_lib = None

_TP = C.POINTER(Tensor)
_vp, _i, _i64, _d, _sz = C.c_void_p, C.c_int, C.c_int64, C.c_double, C.c_size_t

# name -> argtypes, for every zenu_hip_* entry point of include/zenu_hip.h
SIGNATURES = {
    "zenu_hip_init": [_i],
    "zenu_hip_shutdown": [],
    "zenu_hip_last_hip_error": [],
    "zenu_hip_last_status": [],
    "zenu_hip_stream_create": [C.POINTER(_vp)],
    "zenu_hip_stream_destroy": [_vp],
    "zenu_hip_stream_synchronize": [_vp],
    "zenu_hip_device_synchronize": [],
    "zenu_hip_malloc": [C.POINTER(_vp), _sz, _vp],
    "zenu_hip_free": [_vp, _vp],
    "zenu_hip_release_captured": [_vp],
    "zenu_hip_mempool_trim": [],
    "zenu_hip_mempool_stats": [C.POINTER(MempoolStats)],
    "zenu_hip_raw_malloc": [C.POINTER(_vp), _sz],
    "zenu_hip_raw_free": [_vp],
    "zenu_hip_memcpy_h2d": [_vp, _vp, _sz, _vp],
    "zenu_hip_memcpy_d2h": [_vp, _vp, _sz, _vp],
    "zenu_hip_memcpy_d2d": [_vp, _vp, _sz, _vp],
    "zenu_hip_memset_zero": [_vp, _sz, _vp],
    "zenu_hip_binary": [_i, _i, _TP, _TP, _TP, _vp],
    "zenu_hip_binary_assign": [_i, _i, _TP, _TP, _vp],
    "zenu_hip_binary_scalar": [_i, _i, _TP, _TP, _d, _vp],
    "zenu_hip_binary_scalar_assign": [_i, _i, _TP, _d, _vp],
    "zenu_hip_binary_scalar_ptr": [_i, _i, _TP, _TP, _vp, _vp],
    "zenu_hip_binary_scalar_assign_ptr": [_i, _i, _TP, _vp, _vp],
    "zenu_hip_unary": [_i, _i, _TP, _TP, _vp],
    "zenu_hip_unary_assign": [_i, _i, _TP, _vp],
    "zenu_hip_powf": [_i, _TP, _TP, _d, _vp],
    "zenu_hip_relu": [_i, _TP, _TP, _d, _vp],
    "zenu_hip_relu_backward_mask": [_i, _TP, _TP, _d, _vp],
    "zenu_hip_relu_backward": [_i, _TP, _TP, _TP, _d, _vp],
    "zenu_hip_tanh_backward": [_i, _TP, _TP, _TP, _vp],
    "zenu_hip_sigmoid_backward": [_i, _TP, _TP, _TP, _vp],
    "zenu_hip_clip": [_i, _TP, _TP, _d, _d, _vp],
    "zenu_hip_clip_backward_mask": [_i, _TP, _TP, _d, _d, _vp],
    "zenu_hip_copy": [_i, _TP, _TP, _vp],
    "zenu_hip_broadcast": [_i, _TP, _TP, _vp],
    "zenu_hip_softmax": [_i, _TP, _TP, _i, _vp],
    "zenu_hip_softmax_backward": [_i, _TP, _TP, _TP, _i, _vp],
    "zenu_hip_softmax_cross_entropy": [_i, _TP, _TP, _TP, _TP, _vp],
    "zenu_hip_softmax_cross_entropy_backward": [_i, _TP, _TP, _TP, _TP, _vp],
    "zenu_hip_bias_add_relu": [_i, _TP, _TP, _TP, _TP, _d, _vp],
    "zenu_hip_relu_backward_bias_grad": [_i, _TP, _TP, _TP, _TP, _d, _vp],
    "zenu_hip_softmax_cross_entropy_backward_bias_grad": [_i, _TP, _TP, _TP, _TP, _TP, _vp],
    "zenu_hip_sum_axis": [_i, _TP, _TP, _i, _vp],
    "zenu_hip_sum_axis_noalloc": [_i, _TP, _TP, _i, _vp],
    "zenu_hip_set_reduce_spin_limit": [_i],
    "zenu_hip_reduce_fallback_count": [C.POINTER(C.c_uint64)],
    "zenu_hip_selfcheck_short_division": [_i, C.POINTER(C.c_uint64), C.POINTER(C.c_uint32), _vp],
    "zenu_hip_unary_range_hash": [_i, C.c_uint64, C.c_uint64, _i, _vp, _vp],
    "zenu_hip_powf_range_hash": [C.c_double, C.c_uint64, C.c_uint64, _i, _vp, _vp],
    "zenu_hip_unary_range_hash_f64": [_i, C.c_uint64, C.c_uint64, _i, C.c_uint32, C.c_uint32, C.c_uint64, _vp, _vp],
    "zenu_hip_powf_range_hash_f64": [C.c_double, C.c_uint64, C.c_uint64, _i, C.c_uint32, C.c_uint32, C.c_uint64, _vp, _vp],
    "zenu_hip_sum_all": [_i, _vp, _TP, _vp],
    "zenu_hip_sum_to": [_i, _TP, _TP, _vp],
    "zenu_hip_max_axis": [_i, _TP, _TP, _i, _vp],
    "zenu_hip_max_axis_idx": [_i, _vp, _TP, _i, _vp],
    "zenu_hip_max_idx": [_i, _vp, _vp, _TP, _vp],
    "zenu_hip_asum": [_i, _vp, _TP, _vp],
    "zenu_hip_sgd_step": [_i, _vp, _vp, _i64, _d, _vp],
    "zenu_hip_sgd_step_multi": [_i, _i, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i64), _d, _vp],
    "zenu_hip_adam_step": [_i, _vp, _vp, _vp, _vp, _i64, _d, _d, _d, _d, _d, _vp],
    "zenu_hip_adamw_step": [_i, _vp, _vp, _vp, _vp, _i64, _d, _d, _d, _d, _d, _i, _d, _vp],
    "zenu_hip_adam_step_multi": [_i, _i, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                                 C.POINTER(_i64), _d, _d, _d, _d, _d, C.POINTER(C.c_int32), _d, _vp],
    "zenu_hip_adam_schedule_create": [C.POINTER(_vp), _i, _d, _d, _i64, _i, _vp],
    "zenu_hip_adam_schedule_destroy": [_vp, _vp],
    "zenu_hip_adam_schedule_query": [_vp, C.POINTER(_i64), C.POINTER(_i64), C.POINTER(_i64), _vp],
    "zenu_hip_adam_step_multi_scheduled": [_i, _i, C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp),
                                           C.POINTER(_i64), _d, _d, _d, C.POINTER(C.c_int32), _vp, _vp],
}

_BIN = ("add", "sub", "mul", "div")
_UN = ("exp", "log", "tanh", "sqrt", "abs", "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh")


def reference_named_symbols():
    """Names of the 1-D entry points that keep the reference's own names
    (zenu-cuda-kernel-sys/kernel/*.h)."""
    names = []
    for s in ("float", "double"):
        for op in _BIN:
            names += [f"array_array_{op}_{s}", f"array_array_{op}_assign_{s}",
                      f"array_scalar_{op}_{s}", f"array_scalar_{op}_assign_{s}",
                      f"array_scalar_pointer_{op}_{s}", f"array_scalar_pointer_{op}_assign_{s}"]
        for fn in _UN:
            names += [f"array_{fn}_{s}", f"array_{fn}_assign_{s}"]
        names += [f"relu_{s}", f"relu_backward_mask_{s}", f"array_max_idx_{s}",
                  f"memory_access_{s}", f"memory_set_{s}",
                  f"array_clip_{s}", f"array_clip_assign_{s}", f"array_clip_backward_{s}",
                  f"array_clip_backward_assign_{s}", f"conv_bias_add_{s}", f"conv2d_bias_bkwd_{s}",
                  f"array_pow_{s}", f"array_pow_assign_{s}"]
    return names


def lib():
    """Load libzenu_hip.so once and attach argument types."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C zenu_amd/csrc` "
            "(or __graft_entry__.build()); there is no CPU fallback")
    l = C.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(l, name)
        fn.argtypes = args
        fn.restype = C.c_int
    l.zenu_hip_status_string.argtypes = [C.c_int]
    l.zenu_hip_status_string.restype = C.c_char_p
    l.zenu_hip_validated_libm.argtypes = []
    l.zenu_hip_validated_libm.restype = C.c_char_p
    l.zenu_hip_last_hip_error_string.argtypes = []
    l.zenu_hip_last_hip_error_string.restype = C.c_char_p
    _lib = l
    return l


def check(status, where):
    if status != OK:
        l = lib()
        detail = l.zenu_hip_status_string(status).decode()
        if status == ERR_HIP:
            detail += ": " + l.zenu_hip_last_hip_error_string().decode()
        raise ZenuHipError(status, where, detail)
