#!/usr/bin/env python3
"""Benchmark of the device tensor-kernel layer on one MI355X.

A "step" is one pass of the hot path over synthetic inputs: every op of BASELINE.json's
configs[0..3] once (contiguous / broadcast / transposed elementwise, activations, axis
reductions in f32 and f64, one fused AdamW step over 25 M parameters), each on device-resident
buffers.  `value` is whole-step throughput: the algorithmic bytes of one step divided by the
wall time of a step, with K steps timed between two stream synchronisations.

Besides the whole-step figure every op is timed on its own with HIP events recorded on the
stream the kernels are launched on (`ops` in the JSON line), rotating through enough buffer
sets (>= 1 GiB per op) that the 256 MB memory-side cache cannot serve the inputs.  `roofline`
describes the dominant kernel of the step (the fused AdamW update).  `cpu_baseline` is the CPU
oracle (a single-threaded restatement of ZeNu's CPU path, reference-shaped: one leaf loop per
row / slice, whole-array passes with temporaries for Adam) timed on this box's host cores on
one pass of the same step.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload suite|c0|c1|c2|c3|c4|fused]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_HBM_GBPS = 8000.0  # MI355X published HBM3E peak

HP = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, wd=0.01, step=10)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


class Hip:
    """the few HIP runtime calls the harness needs (events), bound with ctypes"""

    def __init__(self):
        self.rt = C.CDLL("libamdhip64.so")
        self.rt.hipEventCreate.argtypes = [C.POINTER(C.c_void_p)]
        self.rt.hipEventRecord.argtypes = [C.c_void_p, C.c_void_p]
        self.rt.hipEventSynchronize.argtypes = [C.c_void_p]
        self.rt.hipEventElapsedTime.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p]

    def event(self):
        e = C.c_void_p()
        assert self.rt.hipEventCreate(C.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.rt.hipEventRecord(e, stream) == 0

    def elapsed_ms(self, a, b):
        assert self.rt.hipEventSynchronize(b) == 0
        ms = C.c_float()
        assert self.rt.hipEventElapsedTime(C.byref(ms), a, b) == 0
        return ms.value


class ClockProbe:
    """The shader clock right after a batch of launches (harness/native/clock_probe.hip: a chain of
    dependent multiply-adds run by one wavefront between the shader-clock counter and the 100 MHz
    constant-rate counter).  None-valued when the helper library is not built."""

    def __init__(self, z, slots=4):
        self.lib = None
        path = os.path.join(ROOT, "harness", "native", "bin", "libclock_probe.so")
        if not os.path.exists(path):
            return
        try:
            lib = C.CDLL(path)
            lib.clock_probe_launch.argtypes = [C.c_void_p, C.c_int, C.c_void_p]
            self.wall_khz = lib.clock_probe_wall_rate_khz()
            self.buf = C.c_void_p()
            if z.lib().zenu_hip_raw_malloc(C.byref(self.buf), 32 * slots) != 0 or self.wall_khz <= 0:
                return
            self.z, self.lib = z, lib
        except OSError:
            self.lib = None

    def sample(self, slot, stream):
        """queue one sample (about 15 us of one wavefront) on `stream`"""
        if self.lib is not None:
            self.lib.clock_probe_launch(C.c_void_p(self.buf.value + 32 * slot), 300, stream)

    def read_mhz(self, n, stream):
        """shader clock in MHz for slots 0..n-1 (after their stream work has finished), or None"""
        if self.lib is None:
            return None
        host = (C.c_uint64 * (4 * n))()
        if self.z.lib().zenu_hip_memcpy_d2h(host, self.buf, 32 * n, stream) != 0:
            return None
        out = []
        for i in range(n):
            c, w = host[4 * i], host[4 * i + 1]
            out.append(round(c / w * self.wall_khz / 1e3, 0) if w else None)
        return out


class Op:
    """one op of the step: a list of pre-bound launch closures, one per rotating buffer set"""

    def __init__(self, name, config, dtype, alg_bytes, elems, launches, cpu_fn, kernel=None):
        self.name, self.config, self.dtype = name, config, dtype
        self.alg_bytes, self.elems = alg_bytes, elems
        self.launches = launches
        self.cpu_fn = cpu_fn
        self.kernel = kernel
        self.i = 0

    def launch(self):
        self.launches[self.i % len(self.launches)]()
        self.i += 1


def build_ops(z, workload, stream):
    """allocate device buffers, upload seeded inputs, return the list of ops"""
    from zenu_amd import _lib
    from zenu_amd._lib import check
    import zenu_oracle as zo

    l = z.lib()
    M = z.Matrix
    ops = []
    GiB = 1 << 30

    def nsets(bytes_per_set):
        return max(2, -(-GiB // bytes_per_set))

    def ref(t):
        return C.byref(t)

    want = lambda c: workload in ("suite", c)

    # ---- config[0]: contiguous f32 [2^24], uniform[-1,1), seed 0 ------------------------------
    def add_c0():
        r = np.random.default_rng(0)
        n = 1 << 24
        a = r.uniform(-1, 1, n).astype(np.float32)
        b = r.uniform(-1, 1, n).astype(np.float32)
        sets = [(M.from_numpy(a), M.from_numpy(b), M.alloc([n])) for _ in range(nsets(3 * 4 * n))]
        keep = sets
        out_h = np.empty_like(a)

        def mk_bin(op):
            ls = []
            for A, B, O in sets:
                da, db, do = A.desc(), B.desc(), O.desc()
                ls.append(lambda da=da, db=db, do=do: check(l.zenu_hip_binary(op, _lib.F32, ref(do), ref(da), ref(db), stream), "binary"))
            return ls
        ops.append(Op("add[2^24]", "c0", "f32", 3 * 4 * n, n, mk_bin(_lib.ADD), lambda: zo.binary_array(zo.ADD, out_h, a, b)))
        ops.append(Op("mul[2^24]", "c0", "f32", 3 * 4 * n, n, mk_bin(_lib.MUL), lambda: zo.binary_array(zo.MUL, out_h, a, b)))
        ls = []
        for A, B, O in sets:
            da, do = A.desc(), O.desc()
            ls.append(lambda da=da, do=do: check(l.zenu_hip_relu(_lib.F32, ref(do), ref(da), 0.0, stream), "relu"))
        ops.append(Op("relu[2^24]", "c0", "f32", 2 * 4 * n, n, ls, lambda: zo.relu(out_h, a, 0.0)))
        ls = []
        for A, B, O in sets:
            da, do = A.desc(), O.desc()
            ls.append(lambda da=da, do=do: check(l.zenu_hip_copy(_lib.F32, ref(do), ref(da), stream), "copy"))
        ops.append(Op("copy[2^24]", "c0", "f32", 2 * 4 * n, n, ls, lambda: zo.copy_from(out_h, a)))
        ops[-1].keep = keep

    # ---- config[1]: [4096,4096] f32, normal(0,1), seed 1 ----------------------------------------
    def add_c1():
        r = np.random.default_rng(1)
        a = r.standard_normal((4096, 4096)).astype(np.float32)
        b = r.standard_normal((4096, 4096)).astype(np.float32)
        row = r.standard_normal((1, 4096)).astype(np.float32)
        n = a.size
        sets = [(M.from_numpy(a), M.from_numpy(b), M.from_numpy(row), M.alloc([4096, 4096])) for _ in range(nsets(3 * 4 * n))]
        out_h = np.empty_like(a)

        def mk(fn):
            return [fn(A.desc(), B.desc(), B.transpose().desc(), R.desc(), O.desc()) for A, B, R, O in sets]
        ops.append(Op("a+b[1,4096]", "c1", "f32", 2 * 4 * n + 4 * 4096, n,
                      mk(lambda da, db, dbt, dr, do: (lambda: check(l.zenu_hip_binary(_lib.ADD, _lib.F32, ref(do), ref(da), ref(dr), stream), "bcast"))),
                      lambda: zo.binary_array(zo.ADD, out_h, a, row)))
        ops.append(Op("a+b^T", "c1", "f32", 3 * 4 * n, n,
                      mk(lambda da, db, dbt, dr, do: (lambda: check(l.zenu_hip_binary(_lib.ADD, _lib.F32, ref(do), ref(da), ref(dbt), stream), "transposed"))),
                      lambda: zo.binary_array(zo.ADD, out_h, a, b.T)))
        ops.append(Op("a*0.5", "c1", "f32", 2 * 4 * n, n,
                      mk(lambda da, db, dbt, dr, do: (lambda: check(l.zenu_hip_binary_scalar(_lib.MUL, _lib.F32, ref(do), ref(da), 0.5, stream), "scalar"))),
                      lambda: zo.binary_scalar(zo.MUL, out_h, a, 0.5)))
        for name, fn, zfn in (("sigmoid", _lib.SIGMOID, None), ("tanh", _lib.TANH, zo.TANH), ("exp", _lib.EXP, zo.EXP)):
            cpu = (lambda: zo.sigmoid(out_h, a)) if zfn is None else (lambda zfn=zfn: zo.unary(zfn, out_h, a))
            ops.append(Op(name, "c1", "f32", 2 * 4 * n, n,
                          mk(lambda da, db, dbt, dr, do, fn=fn: (lambda: check(l.zenu_hip_unary(fn, _lib.F32, ref(do), ref(da), stream), "unary"))),
                          cpu))
        ops[-1].keep = sets

    def add_c2(dt, dcode, dname):
        r = np.random.default_rng(2)
        x = r.standard_normal((8192, 4096)).astype(dt)
        for row in r.choice(8192, size=82, replace=False):
            x[row, int(r.integers(0, 4096))] = x[row].max()
        inb = x.nbytes
        sets = []
        for _ in range(nsets(inb)):
            X = M.from_numpy(x)
            sets.append((X, M.alloc([4096], dt), M.alloc([8192], dt), M.alloc([8192], np.int64), M.alloc([], dt)))
        isz = np.dtype(dt).itemsize
        cpu_all = np.zeros((), dtype=dt)

        def mk(fn):
            return [fn(X.desc(), o0.desc(), o1.desc(), oi.as_ptr(), oa.as_ptr()) for X, o0, o1, oi, oa in sets]
        ops.append(Op(f"sum axis0 {dname}", "c2", dname, inb + 4096 * isz, x.size,
                      mk(lambda dx, d0, d1, pi, pa: (lambda: check(l.zenu_hip_sum_axis(dcode, ref(d0), ref(dx), 0, stream), "sum0"))),
                      lambda: zo.sum_axis(x, 0), kernel=f"reduce_cols_regular_kernel<{'float' if dname == 'f32' else 'double'}, SumTr, {16 // isz}, true>"))
        ops.append(Op(f"sum axis1 {dname}", "c2", dname, inb + 8192 * isz, x.size,
                      mk(lambda dx, d0, d1, pi, pa: (lambda: check(l.zenu_hip_sum_axis(dcode, ref(d1), ref(dx), 1, stream), "sum1"))),
                      lambda: zo.sum_axis(x, 1)))
        ops.append(Op(f"max axis1 {dname}", "c2", dname, inb + 8192 * isz, x.size,
                      mk(lambda dx, d0, d1, pi, pa: (lambda: check(l.zenu_hip_max_axis(dcode, ref(d1), ref(dx), 1, stream), "max1"))),
                      lambda: zo.max_axis(x, 1)))
        ops.append(Op(f"argmax axis1 {dname}", "c2", dname, inb + 8192 * 8, x.size,
                      mk(lambda dx, d0, d1, pi, pa: (lambda: check(l.zenu_hip_max_axis_idx(dcode, pi, ref(dx), 1, stream), "argmax1"))),
                      lambda: zo.max_axis_idx_ravel(x, 1)))
        ops.append(Op(f"sum all {dname}", "c2", dname, inb + isz, x.size,
                      mk(lambda dx, d0, d1, pi, pa: (lambda: check(l.zenu_hip_sum_all(dcode, pa, ref(dx), stream), "sumall"))),
                      lambda: zo.sum_to(x, cpu_all)))
        ops[-1].keep = sets

    # ---- config[2]: [8192,4096] f32 and f64, normal(0,1), seed 2, ~1% duplicate maxima -------------

    # ---- config[3]: fused AdamW over 25 M f32 parameters, seed 3 ---------------------------------------
    def add_c3():
        r = np.random.default_rng(3)
        n = 25_000_000
        p = (r.standard_normal(n) * 0.02).astype(np.float32)
        g = (r.standard_normal(n) * 1e-3).astype(np.float32)
        m = (r.standard_normal(n) * 1e-4).astype(np.float32)
        v = np.abs(r.standard_normal(n) * 1e-6).astype(np.float32)
        sets = [tuple(M.from_numpy(t) for t in (p, g, m, v)) for _ in range(nsets(4 * 4 * n))]
        f = np.float32
        hp = [float(f(HP[k])) for k in ("lr", "beta1", "beta2", "eps", "wd")]
        ls = []
        for P, G, Mm, V in sets:
            ls.append(lambda P=P.as_ptr(), G=G.as_ptr(), Mm=Mm.as_ptr(), V=V.as_ptr(): check(
                l.zenu_hip_adamw_step(_lib.F32, P, G, Mm, V, n, hp[0], hp[1], hp[2], hp[3], hp[4], 1, float(HP["step"]), stream), "adamw"))
        pc, mc, vc = p.copy(), m.copy(), v.copy()
        op = Op("adamw 25M", "c3", "f32", 7 * 4 * n, n, ls,
                lambda: zo.adamw_update(pc, g, mc, vc, f(HP["lr"]), f(HP["beta1"]), f(HP["beta2"]), f(HP["eps"]), f(HP["wd"]), True, f(HP["step"])),
                kernel="adam_kernel<float, 4, true>")
        op.keep = sets
        ops.append(op)

    # ---- not a BASELINE config: the fused entry points at configs[2]'s size, seed 5 ---------------------
    def add_fused():
        r = np.random.default_rng(5)
        shape = (8192, 4096)
        x = r.standard_normal(shape).astype(np.float32)
        t = np.zeros(shape, dtype=np.float32)
        t[np.arange(shape[0]), r.integers(0, shape[1], shape[0])] = 1
        bias = r.standard_normal(shape[1]).astype(np.float32)
        n = x.size
        sets = [(M.from_numpy(x), M.from_numpy(t), M.alloc(shape), M.alloc(shape), M.from_numpy(bias), M.alloc([]))
                for _ in range(nsets(4 * 4 * n))]
        import cpu_matrix   # oracle/: the CPU chains behind the cpu_fn legs
        cx, ct, cb = (cpu_matrix.CpuMatrix.from_numpy(v) for v in (x, t, bias))
        co = cpu_matrix.CpuMatrix.zeros(shape)

        def mk(fn):
            return [fn(X.desc(), T.desc(), O.desc(), P.desc(), B.desc(), L.desc()) for X, T, O, P, B, L in sets]
        ops.append(Op("softmax rows", "fused", "f32", 2 * 4 * n, n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_softmax(_lib.F32, ref(do), ref(dx), 1, stream), "softmax"))),
                      lambda: co.softmax_assign(cx, 1)))
        ops.append(Op("softmax backward", "fused", "f32", 3 * 4 * n, n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_softmax_backward(_lib.F32, ref(do), ref(dp), ref(dx), 1, stream), "softmax_bwd"))),
                      lambda: cpu_matrix.softmax_backward(co, cx, 1)))
        ops.append(Op("softmax cross-entropy", "fused", "f32", 3 * 4 * n, n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_softmax_cross_entropy(_lib.F32, ref(dl), ref(dp), ref(dx), ref(dt), stream), "ce"))),
                      lambda: cpu_matrix.cross_entropy(cx, ct)))
        ops.append(Op("cross-entropy backward", "fused", "f32", 3 * 4 * n, n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_softmax_cross_entropy_backward(_lib.F32, ref(do), ref(dp), ref(dt), None, stream), "ce_bwd"))),
                      lambda: cpu_matrix.cross_entropy_backward(co, ct)))
        ops.append(Op("bias add + relu (2 outputs)", "fused", "f32", 3 * 4 * n + 4 * shape[1], n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_bias_add_relu(_lib.F32, ref(dp), ref(do), ref(dx), ref(db), 0.0, stream), "bias_relu"))),
                      lambda: co.bias_add_relu(cx, cb, 0.0, pre=co)))
        ops.append(Op("relu backward", "fused", "f32", 3 * 4 * n, n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_relu_backward(_lib.F32, ref(do), ref(dt), ref(dx), 0.0, stream), "relu_bwd"))),
                      lambda: co.relu_backward(ct, cx, 0.0)))
        ops.append(Op("clip", "fused", "f32", 2 * 4 * n, n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_clip(_lib.F32, ref(do), ref(dx), -1.0, 1.0, stream), "clip"))),
                      lambda: cx.clip(-1.0, 1.0)))
        ops.append(Op("tanh backward", "fused", "f32", 3 * 4 * n, n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_tanh_backward(_lib.F32, ref(do), ref(dt), ref(dx), stream), "tanh_bwd"))),
                      lambda: co.tanh_backward(ct, cx)))
        ops.append(Op("sigmoid backward", "fused", "f32", 3 * 4 * n, n,
                      mk(lambda dx, dt, do, dp, db, dl: (lambda: check(l.zenu_hip_sigmoid_backward(_lib.F32, ref(do), ref(dt), ref(dx), stream), "sigmoid_bwd"))),
                      lambda: co.sigmoid_backward(ct, cx)))
        ops[-1].keep = sets

    # ---- the neighbours of the path: strided copy / transpose / broadcast, the rest of the unary surface,
    # powf, asum, the bias-gradient reduction (not a BASELINE config) ------------------------------------
    def add_next():
        r = np.random.default_rng(6)
        n = 4096
        a = r.standard_normal((n, n)).astype(np.float32)
        pos = (np.abs(a) + np.float32(0.01)).astype(np.float32)
        unit = np.clip(a, -0.99, 0.99).astype(np.float32)
        row = r.standard_normal(n).astype(np.float32)
        nb = 4 * n * n
        sets = [(M.from_numpy(a), M.from_numpy(pos), M.from_numpy(unit), M.from_numpy(row), M.alloc((n, n)), M.alloc((n,)), M.alloc(()))
                for _ in range(nsets(4 * nb))]
        out_h = np.empty_like(a)
        col_h = np.empty(n, dtype=np.float32)

        def mk(fn):
            return [fn(A, P, U, R, O, V, S) for A, P, U, R, O, V, S in sets]
        ops.append(Op("transpose copy (to_default_stride of a^T)", "next", "f32", 2 * nb, n * n,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=O.desc(), s_=A.transpose().desc(): check(l.zenu_hip_copy(_lib.F32, ref(d), ref(s_), stream), "copy"))),
                      lambda: zo.copy_from(out_h, a.T)))
        ops.append(Op("row-sliced copy (every other row)", "next", "f32", nb, n * n // 2,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=O.slice(slice(0, n // 2)).desc(), s_=A.slice(slice(None, None, 2)).desc(): check(l.zenu_hip_copy(_lib.F32, ref(d), ref(s_), stream), "copy"))),
                      lambda: zo.copy_from(out_h[:n // 2], a[::2])))
        ops.append(Op("broadcast [4096] -> [4096,4096]", "next", "f32", nb + 4 * n, n * n,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=O.desc(), s_=R.desc(): check(l.zenu_hip_broadcast(_lib.F32, ref(d), ref(s_), stream), "broadcast"))),
                      lambda: zo.broadcast(out_h, row)))
        for name, fn, src in (("log", _lib.LOG, 1), ("sqrt", _lib.SQRT, 1), ("abs", _lib.ABS, 0), ("sin", _lib.SIN, 0), ("cos", _lib.COS, 0),
                              ("tan", _lib.TAN, 2), ("asin", _lib.ASIN, 2), ("acos", _lib.ACOS, 2), ("atan", _lib.ATAN, 0),
                              ("sinh", _lib.SINH, 0), ("cosh", _lib.COSH, 0)):
            host = (a, pos, unit)[src]
            ops.append(Op(name, "next", "f32", 2 * nb, n * n,
                          mk(lambda A, P, U, R, O, V, S, fn=fn, src=src: (lambda d=O.desc(), s_=(A, P, U)[src].desc(): check(l.zenu_hip_unary(fn, _lib.F32, ref(d), ref(s_), stream), "unary"))),
                          lambda fn=fn, host=host: zo.unary(fn, out_h, host)))
        # views that none of the contiguous / row / tile kernels take: a strided destination, a gather, and a
        # 4-d permuted copy (NCHW -> NHWC of [64,64,64,64], the tile kernel with two batch dims)
        half = n // 2
        ops.append(Op("out[:, ::2] = a[:, :half] + b[:, :half] (strided destination)", "next", "f32", 3 * nb // 2, n * half,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=O.slice(slice(None), slice(0, n, 2)).desc(), x=A.slice(slice(None), slice(0, half)).desc(),
                                                             y=P.slice(slice(None), slice(0, half)).desc():
                                                      check(l.zenu_hip_binary(_lib.ADD, _lib.F32, ref(d), ref(x), ref(y), stream), "strided dst"))),
                      lambda: zo.binary_array(zo.ADD, out_h[:, ::2], a[:, :half], pos[:, :half])))
        ops.append(Op("out[:, :half] = a[:, ::2] + b[:, :half] (gather)", "next", "f32", 3 * nb // 2, n * half,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=O.slice(slice(None), slice(0, half)).desc(), x=A.slice(slice(None), slice(0, n, 2)).desc(),
                                                             y=P.slice(slice(None), slice(0, half)).desc():
                                                      check(l.zenu_hip_binary(_lib.ADD, _lib.F32, ref(d), ref(x), ref(y), stream), "gather"))),
                      lambda: zo.binary_array(zo.ADD, out_h[:, :half], a[:, ::2], pos[:, :half])))
        a4 = a.reshape(64, 64, 64, 64)
        o4 = out_h.reshape(64, 64, 64, 64)
        ops.append(Op("4-d permuted copy NCHW -> NHWC [64,64,64,64]", "next", "f32", 2 * nb, n * n,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=O.reshape((64, 64, 64, 64)).desc(), s_=A.reshape((64, 64, 64, 64)).transpose_by_index([0, 2, 3, 1]).desc():
                                                      check(l.zenu_hip_copy(_lib.F32, ref(d), ref(s_), stream), "permute"))),
                      lambda: zo.copy_from(o4, a4.transpose(0, 2, 3, 1))))
        ops.append(Op("tanh, the <= 2 ulp variant (ZENU_TANH_ULP2)", "next", "f32", 2 * nb, n * n,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=O.desc(), s_=A.desc(): check(l.zenu_hip_unary(_lib.TANH_ULP2, _lib.F32, ref(d), ref(s_), stream), "unary"))),
                      lambda: zo.unary(zo.TANH, out_h, a)))
        ops.append(Op("powf(x, 2.5)", "next", "f32", 2 * nb, n * n,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=O.desc(), s_=P.desc(): check(l.zenu_hip_powf(_lib.F32, ref(d), ref(s_), 2.5, stream), "powf"))),
                      lambda: zo.powf(out_h, pos, 2.5)))
        ops.append(Op("asum (whole tensor)", "next", "f32", nb + 4, n * n,
                      mk(lambda A, P, U, R, O, V, S: (lambda p_=S.as_ptr(), s_=A.desc(): check(l.zenu_hip_asum(_lib.F32, p_, ref(s_), stream), "asum"))),
                      lambda: zo.asum(a)))
        ops.append(Op("sum_to [4096,4096] -> [4096] (bias gradient)", "next", "f32", nb + 4 * n, n * n,
                      mk(lambda A, P, U, R, O, V, S: (lambda d=V.desc(), s_=A.desc(): check(l.zenu_hip_sum_to(_lib.F32, ref(d), ref(s_), stream), "sum_to"))),
                      lambda: zo.sum_to(a, col_h)))
        ops[-1].keep = sets
        # the f64 side of the unary family ([4096,4096] f64: 128 MiB in, 128 MiB out)
        a64 = a.astype(np.float64)
        out64_h = np.empty_like(a64)
        sets64 = [(M.from_numpy(a64), M.alloc((n, n), dtype=np.float64)) for _ in range(nsets(4 * nb))]
        pos64 = np.abs(a64) + 0.01
        sets64p = [(M.from_numpy(pos64), O) for _, O in sets64]
        for name, fn in (("exp f64", _lib.EXP), ("tanh f64", _lib.TANH), ("sigmoid f64", _lib.SIGMOID), ("sinh f64", _lib.SINH),
                         ("cosh f64", _lib.COSH), ("sin f64", _lib.SIN), ("cos f64", _lib.COS), ("log f64", _lib.LOG)):
            src_sets, src_h = (sets64p, pos64) if fn == _lib.LOG else (sets64, a64)
            ls = [(lambda d=O.desc(), s_=A.desc(), fn=fn: check(l.zenu_hip_unary(fn, _lib.F64, ref(d), ref(s_), stream), "unary f64"))
                  for A, O in src_sets]
            cpu = (lambda: zo.sigmoid(out64_h, a64)) if fn == _lib.SIGMOID else (lambda fn=fn, h=src_h: zo.unary(fn, out64_h, h))
            ops.append(Op(name, "next", "f64", 4 * nb, n * n, ls, cpu))
        ops.append(Op("powf(x, 2.5) f64", "next", "f64", 4 * nb, n * n,
                      [(lambda d=O.desc(), s_=A.desc(): check(l.zenu_hip_powf(_lib.F64, ref(d), ref(s_), 2.5, stream), "powf f64"))
                       for A, O in sets64p],
                      lambda: zo.powf(out64_h, pos64, 2.5)))
        ops[-1].keep = (sets, sets64, sets64p)

    # ---- the same kernels on larger tensors: how much of the distance to the roofline is the fixed
    # cost of a launch at the BASELINE sizes (not a BASELINE config) --------------------------------------
    def add_scaling():
        r = np.random.default_rng(7)
        for mib in (64, 256, 1024):
            n = mib * (1 << 20) // 4
            a = r.standard_normal(n).astype(np.float32)
            sets = [(M.from_numpy(a), M.from_numpy(a), M.alloc([n]), M.alloc(())) for _ in range(max(2, 3072 // (3 * mib)))]
            rows = n // 4096
            out_h = np.empty_like(a)

            def mk(fn):
                return [fn(A, B, O, S) for A, B, O, S in sets]
            ops.append(Op(f"copy {mib} MiB", "scaling", "f32", 2 * 4 * n, n,
                          mk(lambda A, B, O, S: (lambda d=O.desc(), s_=A.desc(): check(l.zenu_hip_copy(_lib.F32, ref(d), ref(s_), stream), "copy"))),
                          lambda: zo.copy_from(out_h, a)))
            ops.append(Op(f"add {mib} MiB", "scaling", "f32", 3 * 4 * n, n,
                          mk(lambda A, B, O, S: (lambda d=O.desc(), x=A.desc(), y=B.desc(): check(l.zenu_hip_binary(_lib.ADD, _lib.F32, ref(d), ref(x), ref(y), stream), "add"))),
                          lambda: zo.binary_array(zo.ADD, out_h, a, a)))
            ops.append(Op(f"sum axis1 [{rows},4096]", "scaling", "f32", 4 * n + 4 * rows, n,
                          mk(lambda A, B, O, S: (lambda d=O.slice(slice(0, rows)).desc(), s_=A.reshape((rows, 4096)).desc(): check(l.zenu_hip_sum_axis(_lib.F32, ref(d), ref(s_), 1, stream), "sum"))),
                          lambda: zo.sum_axis(a.reshape(rows, 4096), 1)))
            ops.append(Op(f"sum axis0 [{rows},4096]", "scaling", "f32", 4 * n + 4 * 4096, n,
                          mk(lambda A, B, O, S: (lambda d=O.slice(slice(0, 4096)).desc(), s_=A.reshape((rows, 4096)).desc(): check(l.zenu_hip_sum_axis(_lib.F32, ref(d), ref(s_), 0, stream), "sum"))),
                          lambda: zo.sum_axis(a.reshape(rows, 4096), 0)))
            ops.append(Op(f"sum all {mib} MiB", "scaling", "f32", 4 * n + 4, n,
                          mk(lambda A, B, O, S: (lambda p_=S.as_ptr(), s_=A.desc(): check(l.zenu_hip_sum_all(_lib.F32, p_, ref(s_), stream), "sum_all"))),
                          lambda: zo.sum_to(a, np.zeros((), dtype=np.float32))))
            ops.append(Op(f"tanh {mib} MiB", "scaling", "f32", 2 * 4 * n, n,
                          mk(lambda A, B, O, S: (lambda d=O.desc(), s_=A.desc(): check(l.zenu_hip_unary(_lib.TANH, _lib.F32, ref(d), ref(s_), stream), "tanh"))),
                          lambda: zo.unary(zo.TANH, out_h, a)))
            ops[-1].keep = sets

    if workload == "scaling":
        add_scaling()
    if workload == "fused":
        add_fused()
    if workload == "next":
        add_next()
    if want("c0"):
        add_c0()
    if want("c1"):
        add_c1()
    if want("c2"):
        add_c2(np.float32, _lib.F32, "f32")
        add_c2(np.float64, _lib.F64, "f64")
    if want("c3"):
        add_c3()
    return ops


def measure_c4(z, args, sync, steps=None):
    """configs[4]: the MLP training step (batch 256, 784-512-512-10, softmax-CE, backward, Adam) as
    ZeNu's op sequence; GEMM on rocBLAS, everything else on this library.  Returns the wall time of
    a step for each way of issuing it and, from one event-instrumented step, the time per kernel
    family."""
    from harness import hip_dev, mlp_step
    x, t, params = mlp_step.make_inputs()
    steps = steps or args.steps

    class A:      # what the helpers read
        pass
    a = A()
    a.steps, a.warmup = steps, args.warmup

    def measure(fused):
        dev = hip_dev.HipDev(z, timed=False)
        st = mlp_step.MlpStep(dev, x, t, params, fused=fused)
        for _ in range(max(a.warmup, 3)):
            st.step()
        sync()
        t0 = time.perf_counter()
        for _ in range(steps):
            st.step()
        sync()
        ms = (time.perf_counter() - t0) / steps * 1e3
        dev.__init__(z, timed=True)
        dev.begin()
        st.step()
        br = {k: round(v, 1) for k, v in dev.breakdown().items()}
        return ms, br, capture_and_replay_c4(z, st, a, sync)

    ms, br, graph = measure(False)
    fms, fbr, fgraph = measure(True)
    fused = {"what": "the same step through the fused entry points (bias add + ReLU, softmax cross-entropy "
                     "forward / backward, ReLU backward)",
             "ms_per_step": round(fms, 4), "steps_per_s": round(1e3 / fms, 1),
             "breakdown_us_one_instrumented_step": fbr, "hip_graph_replay": fgraph}
    compiled = compiled_host_c4(x, t, params, a)
    cpu = None
    if not args.no_cpu_baseline:
        import cpu_dev      # oracle/: the CPU leg of the same step
        cst = mlp_step.MlpStep(cpu_dev.CpuDev(), x, t, params)
        cst.step()
        t1 = time.perf_counter()
        n = 3
        for _ in range(n):
            cst.step()
        cpu = dict(value=round(n / (time.perf_counter() - t1), 2), unit="steps/s", cores=1, kind="port",
                   sample=f"{n} steps of the same op sequence on the C oracle (GEMM: numpy/OpenBLAS, its own threads)")
    # headline: ZeNu's op sequence issued by the compiled host when it is built, else by the Python mirror
    head_ms, host = ms, "python mirror (ctypes)"
    if isinstance(compiled.get("ops"), dict) and "ms_per_step" in compiled["ops"]:
        head_ms, host = compiled["ops"]["ms_per_step"], "compiled host (C++ API)"
    return dict(head_ms=head_ms, host=host, ms=ms, breakdown=br, graph=graph, fused=fused, compiled=compiled, cpu=cpu)


C4_WORKLOAD = "configs[4]: batch 256, Linear 784-512-ReLU-512-ReLU-10, softmax-CE, Adam"


def run_c4(z, args, sync):
    """--workload c4: the MLP step as the headline of its own JSON line"""
    r = measure_c4(z, args, sync)
    print(json.dumps({
        "metric": "MLP training step (configs[4]): steps/s; time per kernel family", "value": round(1e3 / r["head_ms"], 1),
        "unit": "steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(r["head_ms"], 4),
        "host": r["host"], "python_mirror_ms_per_step": round(r["ms"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": C4_WORKLOAD},
        "breakdown_us_one_instrumented_step": r["breakdown"], "hip_graph_replay": r["graph"], "fused_entry_points": r["fused"],
        "compiled_host": r["compiled"], "cpu_baseline": r["cpu"]}))


def _launches(graph_result):
    n = graph_result.get("graph_nodes_per_step") if isinstance(graph_result, dict) else None
    return n - 1 if n else None


def c4_summary(z, args, sync):
    """configs[4] for the default line: never `value`, never `roofline`; an object of its own"""
    try:
        r = measure_c4(z, args, sync, steps=max(args.steps, 50))
    except Exception as e:      # the configs[0..3] figures stand on their own
        return {"workload": C4_WORKLOAD, "error": repr(e)}
    comp = r["compiled"]

    def ms_of(key):
        v = comp.get(key) if isinstance(comp, dict) else None
        return v.get("ms_per_step") if isinstance(v, dict) else None
    return {
        "workload": C4_WORKLOAD, "dtype": "f32", "unit": "ms per training step",
        "eager_compiled_host_ms_per_step": ms_of("ops"),
        # the part of it the host needs just to issue the launches (it runs ahead of the GPU): when this is
        # close to the step time the step is bound by the host's per-launch cost, not by the kernels
        "eager_compiled_host_issue_ms_per_step": (comp.get("ops") or {}).get("host_issue_ms_per_step") if isinstance(comp, dict) else None,
        "fused_compiled_host_issue_ms_per_step": (comp.get("fused") or {}).get("host_issue_ms_per_step") if isinstance(comp, dict) else None,
        # one-element adds issued back to back through the C ABI: the cost of a launch as such
        "smallest_launch_us": (comp.get("floor") or {}).get("launch_us") if isinstance(comp, dict) else None,
        "fused_compiled_host_ms_per_step": ms_of("fused"),
        "fused_transposed_views_compiled_host_ms_per_step": ms_of("lean"),
        "eager_python_mirror_ms_per_step": round(r["ms"], 4),
        "fused_python_mirror_ms_per_step": r["fused"]["ms_per_step"],
        "eager_hip_graph_replay": r["graph"], "fused_hip_graph_replay": r["fused"]["hip_graph_replay"],
        "kernel_family_us_eager_step": r["breakdown"],
        "kernel_family_us_fused_step": r["fused"]["breakdown_us_one_instrumented_step"],
        # launches of one eager step = the nodes of its recorded graph minus the cursor advance of the scheduled update
        "launches_per_step": {"eager": _launches(r["graph"]), "fused": _launches(r["fused"]["hip_graph_replay"])},
        "compiled_host_error": comp.get("error") if isinstance(comp, dict) else None,
        "cpu_baseline": r["cpu"],
        "note": "GEMMs on rocBLAS; gemm is one family of the breakdown, every other family is this library; "
                "event-instrumented steps include one event record per op",
    }


def compiled_host_c4(x, t, params, args):
    """The same step issued eagerly from a C++ host (harness/native/mlp_step_bench.cpp, built by
    __graft_entry__.build()): wall time per step without the Python mirror's per-call cost."""
    import subprocess
    import tempfile
    exe = os.path.join(ROOT, "harness", "native", "bin", "mlp_step_bench")
    if not os.path.exists(exe):
        return {"error": "harness/native/bin/mlp_step_bench is not built"}
    with tempfile.TemporaryDirectory() as d:
        path = os.path.join(d, "inputs.bin")
        with open(path, "wb") as f:
            for a in [x, t] + [params[f"linear{i}.{n}"] for i in (1, 2, 3) for n in ("weight", "bias")]:
                f.write(np.ascontiguousarray(a, dtype=np.float32).tobytes())
        out = subprocess.run([exe, "--inputs", path, "--steps", str(max(args.steps, 50)), "--warmup", "5"],
                             capture_output=True, text=True, timeout=120)
    if out.returncode != 0:
        return {"error": (out.stdout + out.stderr)[-300:]}
    res = {}
    for line in out.stdout.splitlines():
        w = line.split()
        if len(w) == 3 and w[1] in ("ms_per_step", "host_issue_ms_per_step", "final_loss", "launch_us"):
            res.setdefault(w[0], {})[w[1]] = float(w[2])
    return res


def capture_and_replay_c4(z, st, args, sync):
    """Capture one whole step (62 launches, 37 with the fused entry points, all on the library's stream, all allocations
    served by the caching pool) into a HIP graph and time its replays: the step without the
    host's per-launch cost.  The recorded Adam update is the scheduled one, so consecutive replays are
    consecutive training steps; the first three are checked bit for bit against three eager steps."""
    import numpy as np
    rt = C.CDLL("libamdhip64.so")
    stream = z.get_stream()
    vp = C.c_void_p
    rt.hipStreamBeginCapture.argtypes = [vp, C.c_int]
    rt.hipStreamEndCapture.argtypes = [vp, C.POINTER(vp)]
    rt.hipGraphInstantiate.argtypes = [C.POINTER(vp), vp, vp, vp, C.c_size_t]
    rt.hipGraphLaunch.argtypes = [vp, vp]
    try:
        dev = st.dev
        dev.timed = False

        def snapshot():
            return ({k: v.to_numpy() for k, v in st.p.items()}, {k: v.to_numpy() for k, v in st.opt.m.items()},
                    {k: v.to_numpy() for k, v in st.opt.v.items()}, st.opt.step)

        def restore(s):
            from zenu_amd import _lib
            for src, dst in ((s[0], st.p), (s[1], st.opt.m), (s[2], st.opt.v)):
                for k, a in src.items():
                    _lib.check(z.lib().zenu_hip_memcpy_h2d(dst[k].as_ptr(), a.ctypes.data, a.nbytes, stream), "h2d")
            st.opt.step = s[3]

        s0 = snapshot()
        eager = []
        for _ in range(3):      # three consecutive eager steps: the reference results, and the rehearsal that
            eager_loss, rehearsal = st.step()   # leaves every block the capture will ask the pool for
            eager.append((float(eager_loss.to_numpy()), {k: v.to_numpy() for k, v in st.p.items()}))
            del rehearsal
        restore(s0)
        # Adam's step advances on every update (adam.rs:21-25): the recorded update takes 1 - beta^t from a
        # table in device memory whose cursor it advances, so replay i is step i
        st.opt.use_schedule(args.steps + 16)
        sync()
        if rt.hipStreamBeginCapture(stream, 2) != 0:   # hipStreamCaptureModeRelaxed
            return {"error": "hipStreamBeginCapture failed"}
        g = vp()
        try:
            loss, grads = st.step()                     # recorded, not executed
        finally:
            rc = rt.hipStreamEndCapture(stream, C.byref(g))
        if rc != 0:
            return {"error": "hipStreamEndCapture failed"}
        n_nodes = C.c_size_t(0)
        rt.hipGraphGetNodes.argtypes = [vp, vp, C.POINTER(C.c_size_t)]
        if rt.hipGraphGetNodes(g, None, C.byref(n_nodes)) != 0:
            n_nodes = C.c_size_t(0)
        ge = vp()
        if rt.hipGraphInstantiate(C.byref(ge), g, None, None, 0) != 0:
            return {"error": "hipGraphInstantiate failed"}
        checks = 0
        for i in range(3):                              # consecutive replays = consecutive steps, each checked
            assert rt.hipGraphLaunch(ge, stream) == 0
            sync()
            ok = float(loss.to_numpy()) == eager[i][0] and all(np.array_equal(st.p[k].to_numpy(), eager[i][1][k]) for k in st.p)
            if not ok:
                return {"error": f"graph replay {i} differs from eager step {i}"}
            checks += 1
        sync()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            rt.hipGraphLaunch(ge, stream)
        sync()
        ms = (time.perf_counter() - t0) / args.steps * 1e3
        nxt, left, refused = st.opt.schedule_state()
        st.opt.drop_schedule()
        return {"ms_per_step": round(ms, 4), "steps_per_s": round(1e3 / ms, 1), "consecutive_steps_checked_bit_exact": checks,
                "adam_step": "advances on the device with every replay (scheduled update)", "steps_taken": nxt - 1,
                "updates_refused": refused,
                # counted from the recorded graph: every launch of one step, the one-thread launch that
                # advances the schedule's cursor included (an eager step does not have that one)
                "graph_nodes_per_step": n_nodes.value or None}
    except Exception as e:  # the eager figures above stand on their own
        return {"error": repr(e)}


# ops whose HBM traffic was measured with rocprofv3 --pmc: op name -> (summary under profiles/, the
# sources that define the op's kernel).  A summary records the hash of those sources at the time of
# the counter run; if the kernel's sources have changed since, the figure is stale and not reported.
TRAFFIC_PROFILES = {
    "adamw 25M": ("adam_kernel_c3_adamw25M_pmc_traffic.txt",
                  ("zenu_amd/csrc/optim.hip", "zenu_amd/csrc/vecmem.hpp", "zenu_amd/csrc/common.hpp")),
    "sum axis0 f64": ("reduce_cols_regular_kernel_c2_sum_axis0_f64_pmc_traffic.txt",
                      ("zenu_amd/csrc/reduce.hip", "zenu_amd/csrc/vecmem.hpp", "zenu_amd/csrc/common.hpp")),
}


def kernel_sources_sha256(paths):
    import hashlib
    h = hashlib.sha256()
    for rel in paths:
        with open(os.path.join(ROOT, rel), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def measured_traffic(op):
    """(HBM bytes per launch of the op's kernel, note): FETCH_SIZE + WRITE_SIZE from the committed
    rocprofv3 --pmc summary, each scaled by what the same counter reads for a copy kernel of known
    size; (None, reason) when no summary exists or the kernel's sources have changed since it was made."""
    if op.name not in TRAFFIC_PROFILES:
        return None, "no counter run recorded for this op"
    fname, sources = TRAFFIC_PROFILES[op.name]
    fields = {}
    try:
        for line in open(os.path.join(ROOT, "profiles", fname)):
            if ":" in line:
                k, v = line.split(":", 1)
                fields[k.strip()] = v.strip()
    except OSError:
        return None, f"profiles/{fname} is missing"
    if "traffic_bytes_per_launch" not in fields:
        return None, f"profiles/{fname} holds no traffic figure"
    if fields.get("kernel_sources_sha256") != kernel_sources_sha256(sources):
        return None, f"profiles/{fname} was made from other kernel sources ({', '.join(sources)} changed since): stale, not reported"
    return int(fields["traffic_bytes_per_launch"]), f"profiles/{fname}"


def roofline_of(row, op):
    traffic, note = measured_traffic(op)
    return dict(bound="hbm", achieved=row["GBps"], peak=PEAK_HBM_GBPS, unit="GB/s",
                frac=round(row["GBps"] / PEAK_HBM_GBPS, 4), traffic=traffic, traffic_source=note,
                kernel=op.kernel or row["op"], op=row["op"], algorithmic_bytes_per_launch=row["alg_bytes"],
                avg_launch_us=row["us"])


def time_ops(ops, args, hip, stream, sync, probe, bracketed=True):
    """Per-op timing with HIP events on the launch stream.
    Three batches of op_reps back-to-back launches, one event pair around each; `us` is the median
    of the three batch means (kernels bound by their vector instructions follow the clock, which the
    power management moves by +-10 % from one millisecond to the next; `us_batches` keeps all three,
    `shader_mhz_batches` the clock sampled right after each batch) and agrees with the kernel durations
    of a rocprofv3 trace; a second pass brackets every launch with its own events for a median and a
    minimum, which include the cost of one event record (~2.5 us)."""
    e0, e1 = hip.event(), hip.event()
    marks = [hip.event() for _ in range(args.op_reps + 1)] if bracketed else []
    table = []
    for o in ops:
        for _ in range(10):
            o.launch()
        sync()
        batches = []
        for b in range(3):
            hip.record(e0, stream)
            for _ in range(args.op_reps):
                o.launch()
            hip.record(e1, stream)
            probe.sample(b, stream)
            batches.append(hip.elapsed_ms(e0, e1) / args.op_reps * 1e3)
        mhz = probe.read_mhz(3, stream)
        us = sorted(batches)[1]
        gbps = o.alg_bytes / (us * 1e-6) / 1e9
        row = dict(op=o.name, config=o.config, dtype=o.dtype, us=round(us, 2), GBps=round(gbps, 1),
                   frac_of_peak=round(gbps / PEAK_HBM_GBPS, 4), Gelem_per_s=round(o.elems / (us * 1e-6) / 1e9, 2),
                   alg_bytes=o.alg_bytes, us_batches=[round(b, 2) for b in batches], shader_mhz_batches=mhz)
        if bracketed:
            hip.record(marks[0], stream)
            for i in range(args.op_reps):
                o.launch()
                hip.record(marks[i + 1], stream)
            each = sorted(hip.elapsed_ms(marks[i], marks[i + 1]) * 1e3 for i in range(args.op_reps))
            row.update(us_bracketed_median=round(each[len(each) // 2], 2), us_bracketed_min=round(each[0], 2))
        table.append(row)
        log(f"[op] {o.name:22s} {us:9.2f} us  {gbps:8.1f} GB/s  {100 * gbps / PEAK_HBM_GBPS:5.1f}% of peak  clock {mhz}")
    return table


def extra_rows(z, workload, args, hip, stream, sync, probe):
    """the rows that come after the BASELINE configs, compact, for the default line: op -> [us, % of peak,
    shader MHz of the median batch]; never `value`, never `roofline`, no CPU leg"""
    try:
        t0 = time.time()
        ops = build_ops(z, workload, stream)
        sync()
        rows = time_ops(ops, args, hip, stream, sync, probe, bracketed=False)
        out = {}
        for r in rows:
            mid = sorted(range(3), key=lambda i: r["us_batches"][i])[1]
            mhz = r["shader_mhz_batches"][mid] if r["shader_mhz_batches"] else None
            out[r["op"]] = [r["us"], round(100 * r["frac_of_peak"], 1), mhz]
        del ops
        log(f"[{workload}] {len(out)} ops measured in {time.time() - t0:.1f} s")
        return {"columns": ["us per launch (median of 3 batches)", "% of the 8 TB/s HBM peak by algorithmic bytes",
                            "shader clock in MHz right after that batch"], "ops": out}
    except Exception as e:      # the configs[0..3] figures stand on their own
        return {"error": repr(e)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="suite", choices=["suite", "c0", "c1", "c2", "c3", "c4", "fused", "next", "scaling"])
    ap.add_argument("--op-reps", type=int, default=50, help="launches per op in the per-op timing")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-c4", action="store_true", help="leave configs[4] out of the default line (profiling runs)")
    ap.add_argument("--profile-op", default=None, help="only launch this op (for rocprofv3 counter runs)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every op of the path would shard without communication, "
                 "but no multi-GPU path exists): run with --gpus 1")

    import zenu_amd as z
    from zenu_amd import _lib
    _lib.check(z.lib().zenu_hip_init(0), "zenu_hip_init")
    sys.path.insert(0, os.path.join(ROOT, "oracle"))

    stream = C.c_void_p()
    _lib.check(z.lib().zenu_hip_stream_create(C.byref(stream)), "stream_create")
    z.set_stream(stream)
    hip = Hip()
    sync = lambda: _lib.check(z.lib().zenu_hip_stream_synchronize(stream), "sync")

    if args.workload == "c4":
        return run_c4(z, args, sync)
    probe = ClockProbe(z)

    t0 = time.time()
    ops = build_ops(z, args.workload, stream)
    sync()
    log(f"[bench] {len(ops)} ops set up in {time.time() - t0:.1f} s")

    if args.profile_op:
        sel = [o for o in ops if o.name == args.profile_op]
        assert sel, [o.name for o in ops]
        for _ in range(args.warmup + args.steps):
            sel[0].launch()
        sync()
        return

    # ---- whole-step timing -------------------------------------------------------------------------
    for _ in range(args.warmup):
        for o in ops:
            o.launch()
    sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        for o in ops:
            o.launch()
    sync()
    elapsed = time.perf_counter() - t0
    step_bytes = sum(o.alg_bytes for o in ops)
    ms_per_step = elapsed / args.steps * 1e3
    value = step_bytes / (elapsed / args.steps) / 1e9

    table = time_ops(ops, args, hip, stream, sync, probe)

    # dominant kernel of the step = the op with the largest share of the step time
    by_time = sorted(table, key=lambda t: -t["us"])
    dom = by_time[0]
    roofline = roofline_of(dom, [o for o in ops if o.name == dom["op"]][0])
    # the same figures for the second-largest op of the step
    roofline_second = roofline_of(by_time[1], [o for o in ops if o.name == by_time[1]["op"]][0]) if len(by_time) > 1 else None
    adam = [t for t in table if t["config"] == "c3"]

    # ---- CPU baseline: the oracle, one thread, one pass of the same step -----------------------------------
    cpu = None
    if not args.no_cpu_baseline:
        t0 = time.perf_counter()
        per_op = {o.name: 0.0 for o in ops}
        passes = 0
        while passes < 5 and (passes == 0 or time.perf_counter() - t0 < 10.0):
            for o in ops:
                t1 = time.perf_counter()
                o.cpu_fn()
                per_op[o.name] += time.perf_counter() - t1
            passes += 1
        cpu_s = (time.perf_counter() - t0) / passes
        per_op = {k: v / passes for k, v in per_op.items()}
        for t in table:
            t["cpu_GBps"] = round(t["alg_bytes"] / per_op[t["op"]] / 1e9, 3)
        cpu = dict(value=round(step_bytes / cpu_s / 1e9, 3), unit="GB/s", cores=1, kind="port",
                   sample=f"{passes} full pass(es) of the step ({len(ops)} ops, {cpu_s:.1f} s each) by the single-threaded C oracle, "
                          f"reference-shaped (one leaf loop per row/slice, Adam as whole-array passes); "
                          f"host has {os.cpu_count()} logical CPUs")
        log(f"[cpu] one step on the CPU oracle: {cpu_s:.2f} s = {cpu['value']} GB/s")

    # ---- configs[4], the MLP training step: its own object on the default line ---------------------------
    c4 = None
    if args.workload == "suite" and not args.no_c4:
        t0 = time.time()
        c4 = c4_summary(z, args, sync)
        log(f"[c4] MLP step measured in {time.time() - t0:.1f} s: "
            f"{c4.get('eager_compiled_host_ms_per_step')} ms eager, {c4.get('fused_compiled_host_ms_per_step')} ms fused")

    # ---- the rows after the BASELINE configs: compact objects on the default line ---------------------------
    nxt = fused = None
    if args.workload == "suite" and not args.no_c4:
        del ops
        nxt = extra_rows(z, "next", args, hip, stream, sync, probe)
        fused = extra_rows(z, "fused", args, hip, stream, sync, probe)

    out = {
        "metric": "achieved HBM GB/s (% of MI355X peak) per op; Adam step params/sec",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32" if args.workload not in ("suite", "c2", "next") else "f32+f64", "data": "synthetic",
        "config": {"workload": {"suite": "configs[0..3]: every op once per step", "c0": "configs[0]", "c1": "configs[1]",
                                "c2": "configs[2]", "c3": "configs[3]",
                                "fused": "fused entry points on [8192,4096] f32 (not a BASELINE config)",
                                "scaling": "copy, add, sums and tanh on 64 MiB, 256 MiB and 1 GiB f32 tensors (not a BASELINE config)",
                                "next": "strided copy, broadcast, the remaining unary functions, powf, asum and sum_to on [4096,4096] f32, "
                                        "and exp / tanh / sigmoid / sinh / cosh on [4096,4096] f64 (not a BASELINE config)"}[args.workload],
                   "ops_per_step": len(table), "algorithmic_bytes_per_step": step_bytes},
        "frac_of_peak_whole_step": round(value / PEAK_HBM_GBPS, 4),
        "adam_step_params_per_sec": (round(adam[0]["Gelem_per_s"] * 1e9) if adam else None),
        "roofline": roofline, "roofline_second_largest_op": roofline_second, "cpu_baseline": cpu, "c4": c4, "next": nxt, "fused": fused, "ops": table,
        "timing": f"HIP events on the launch stream; per op 3 batches of {args.op_reps} back-to-back launches after 10 warm-up launches: "
                  "us = median of the 3 batch means (us_batches), us_bracketed_* = per-launch event pairs (each includes one event record); "
                  "shader_mhz_batches = the shader clock sampled by a one-wavefront kernel right after each batch",
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
