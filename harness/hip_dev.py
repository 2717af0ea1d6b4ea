"""The HIP device of the MLP step (harness/mlp_step.py): zenu_amd.Matrix and the fused entry
points, GEMM on rocBLAS sgemm / dgemm (the library path, as ZeNu calls cuBLAS).  `tick` lets the
caller attribute time to kernel families with HIP events on the launch stream."""
import ctypes as C

import numpy as np


class HipDev:
    """categories are timed with HIP events on the launch stream when `timed` is set"""

    def __init__(self, hip, timed=False):
        self.hip = hip
        self.M = hip.Matrix
        self.sum_to = hip.sum_to
        self.F = hip             # the fused entry points
        self.blas = C.CDLL("librocblas.so")
        self.handle = C.c_void_p()
        assert self.blas.rocblas_create_handle(C.byref(self.handle)) == 0
        assert self.blas.rocblas_set_stream(self.handle, C.c_void_p(_as_int(hip.get_stream()))) == 0
        self.timed = timed
        self.marks = []
        if timed:
            self.rt = C.CDLL("libamdhip64.so")
            self.rt.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
            self.rt.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
            self.rt.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]
            self.rt.hipEventSynchronize.argtypes = [C.c_void_p]
            self.pool = []

    def _event(self):
        e = C.c_void_p()
        assert self.rt.hipEventCreate(C.byref(e)) == 0
        return e

    def begin(self):
        self.marks = []
        if self.timed:
            self.tick("start")

    def tick(self, category):
        if not self.timed:
            return
        i = len(self.marks)
        if i >= len(self.pool):
            self.pool.append(self._event())
        self.rt.hipEventRecord(self.pool[i], C.c_void_p(_as_int(self.hip.get_stream())))
        self.marks.append(category)

    def breakdown(self):
        """microseconds per category between consecutive ticks of the last step"""
        out = {}
        self.rt.hipEventSynchronize(self.pool[len(self.marks) - 1])
        for i in range(1, len(self.marks)):
            ms = C.c_float()
            self.rt.hipEventElapsedTime(C.byref(ms), self.pool[i - 1], self.pool[i])
            out[self.marks[i]] = out.get(self.marks[i], 0.0) + ms.value * 1e3
        return out

    def gemm(self, a, b):
        """row-major C[m,n] = A[m,k] B[k,n] through column-major rocBLAS: C^T = B^T A^T"""
        m, k = a.shape
        k2, n = b.shape
        assert k == k2 and a.is_default_stride_strict() and b.is_default_stride_strict()
        out = self.M.alloc([m, n], a.dtype)
        if a.dtype == np.float32:
            fn, ct = self.blas.rocblas_sgemm, C.c_float
        else:
            fn, ct = self.blas.rocblas_dgemm, C.c_double
        alpha, beta = ct(1.0), ct(0.0)
        NONE = 111  # rocblas_operation_none
        rc = fn(self.handle, NONE, NONE, n, m, k, C.byref(alpha), C.c_void_p(b.as_ptr()), n, C.c_void_p(a.as_ptr()), k,
                C.byref(beta), C.c_void_p(out.as_ptr()), n)
        assert rc == 0, rc
        return out

    def make_adam(self, params):
        return self.hip.Adam(1e-3, 0.9, 0.999, 1e-8, params)


def _as_int(stream):
    if stream is None:
        return 0
    return stream.value if hasattr(stream, "value") else int(stream)
