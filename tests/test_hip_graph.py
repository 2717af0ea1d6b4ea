"""The library's calls inside a captured HIP graph.

What a capturing caller relies on: no entry point synchronises or calls the driver's allocator
when the caching pool can serve the request (rehearsal runs make every request a hit), zero fills
are kernels (no memset nodes), the arrival counters of the split reductions are back at zero after
every run, and memory taken from the pool during the capture -- the library's scratch as well as
tensors the sequence allocates and drops -- stays out of ordinary requests afterwards, so tensors
allocated after the capture survive every replay.  The graph is replayed several times with new
inputs, eager work on the same stream and synchronisations in between, and every replay is compared
bit for bit with the eager sequence on the same inputs.
"""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _hip_runtime():
    rt = C.CDLL("libamdhip64.so")
    vp = C.c_void_p
    rt.hipStreamBeginCapture.argtypes = [vp, C.c_int]
    rt.hipStreamEndCapture.argtypes = [vp, C.POINTER(vp)]
    rt.hipGraphInstantiate.argtypes = [C.POINTER(vp), vp, vp, vp, C.c_size_t]
    rt.hipGraphLaunch.argtypes = [vp, vp]
    rt.hipGraphExecDestroy.argtypes = [vp]
    rt.hipGraphDestroy.argtypes = [vp]
    return rt


def test_library_calls_in_a_captured_graph(hip):
    import os
    from zenu_amd import _lib
    if os.environ.get("ZENU_USE_MEMPOOL") == "0":
        pytest.skip("without the pool every scratch request is a driver allocation, which cannot be captured")
    rt = _hip_runtime()
    l = hip.lib()
    M = hip.Matrix
    stream = C.c_void_p()
    _lib.check(l.zenu_hip_stream_create(C.byref(stream)), "stream_create")
    old = hip.get_stream()
    hip.set_stream(stream)
    graph, gexec = C.c_void_p(), C.c_void_p()
    try:
        r = np.random.default_rng(41)
        rows, cols = 1024, 2048
        inputs = [r.standard_normal((rows, cols)).astype(np.float32) * s for s in (1.0, 0.5, 2.0, 1.5)]
        t = np.zeros((rows, cols), dtype=np.float32)
        t[np.arange(rows), r.integers(0, cols, rows)] = 1
        x, tgt = M.from_numpy(inputs[0]), M.from_numpy(t)
        bias = M.from_numpy(r.standard_normal(cols).astype(np.float32))
        act, pre, th = M.alloc((rows, cols)), M.alloc((rows, cols)), M.alloc((rows, cols))
        colsum, total = M.alloc((cols,)), M.alloc(())
        argmax = M.alloc((rows,))
        p0 = r.standard_normal(rows * cols).astype(np.float32) * 0.02
        p = M.from_numpy(p0)
        params = {"w": (p, act)}                       # the activations double as a gradient
        opt = hip.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, params, ["w"])
        outs = {}

        def sequence():
            act.bias_add_relu(x, bias, 0.0, pre=pre)            # fused elementwise, two outputs
            th.tanh_array(pre)                                  # exact tanh (VALU path)
            hip.sum_to(act, colsum)                             # split column reduction: scratch + counters
            l.zenu_hip_memset_zero(total.as_ptr(), 4, stream)   # a zero fill inside the capture
            _lib.check(l.zenu_hip_sum_all(_lib.F32, total.as_ptr(), C.byref(x.desc()), stream), "sum_all")
            argmax.copy_from(x.max_axis(1))                     # allocation + arg-max + strided copy
            outs["loss"], outs["prob"] = hip.cross_entropy(x, tgt)
            outs["g"] = hip.cross_entropy_backward(outs["prob"], tgt)
            opt.update(params)

        def state():
            hip.synchronize()
            return [v.to_numpy().copy() for v in (act, pre, th, colsum, total, argmax, outs["loss"], outs["prob"],
                                                  outs["g"], p, opt.m["w"], opt.v["w"])]

        def reset(inp):
            _lib.check(l.zenu_hip_memcpy_h2d(x.as_ptr(), inp.ctypes.data, inp.nbytes, stream), "h2d")
            _lib.check(l.zenu_hip_memcpy_h2d(p.as_ptr(), p0.ctypes.data, p0.nbytes, stream), "h2d")
            for mv in (opt.m["w"], opt.v["w"]):
                _lib.check(l.zenu_hip_memset_zero(mv.as_ptr(), p0.nbytes, stream), "zero")
            opt.step = 0

        eager = []
        for inp in inputs:                                       # also the rehearsal: the pool holds every block
            reset(inp)
            sequence()
            eager.append(state())
        reset(inputs[0])
        hip.synchronize()
        assert rt.hipStreamBeginCapture(stream, 2) == 0          # hipStreamCaptureModeRelaxed
        try:
            sequence()                                           # recorded, not executed
        finally:
            rc = rt.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0
        assert rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        keep = dict(outs)                                        # the captured outputs' buffers
        # tensors allocated AFTER the capture, of every size the sequence used for scratch and
        # temporaries: the recorded kernels still write those addresses on each replay, so none of
        # these may have been given one of them
        sentinel_shapes = [(rows, cols), (rows, cols), (rows, cols), (cols,), (rows,), (), (512, cols), (64, cols),
                           (8, cols), (2 * rows,), (4 * rows,), (130,), (rows * 4,), (cols * 16,), (1 << 20,), (1 << 18,)]
        sentinels = []
        for k, shp in enumerate(sentinel_shapes * 2):
            v = np.full(shp, 1000.0 + k, dtype=np.float32)
            sentinels.append((v, M.from_numpy(v)))
        st0 = _lib.MempoolStats()
        _lib.check(l.zenu_hip_mempool_stats(C.byref(st0)), "stats")
        for i, inp in enumerate(inputs):
            reset(inp)
            opt.step = 1                                         # frozen in the graph as a kernel argument
            assert rt.hipGraphLaunch(gexec, stream) == 0
            got = state()
            for name, a, b in zip(("act", "pre", "tanh", "colsum", "total", "argmax", "loss", "prob", "g", "p", "m", "v"),
                                  got, eager[i]):
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (i, name)
            # eager work between replays: other launches that use counters and pool blocks
            y = (x + x).sum(0)
            z = x.exp().max_axis(1)
            del y, z
            hip.synchronize()
            for v, S in sentinels:
                assert np.array_equal(S.to_numpy(), v), ("a tensor allocated after the capture was overwritten by replay", i, v.shape)
        del keep, sentinels
        hip.synchronize()
        rt.hipGraphExecDestroy(gexec)
        rt.hipGraphDestroy(graph)
        gexec, graph = C.c_void_p(), C.c_void_p()
        _lib.check(l.zenu_hip_release_captured(stream), "release_captured")   # the graph is gone: blocks are ordinary again
        big = [M.alloc((rows, cols)) for _ in range(8)]
        st1 = _lib.MempoolStats()
        _lib.check(l.zenu_hip_mempool_stats(C.byref(st1)), "stats")
        assert st1.bytes_reserved == st1.bytes_in_use + st1.bytes_cached
        del big
    finally:
        hip.synchronize()
        if gexec:
            rt.hipGraphExecDestroy(gexec)
        if graph:
            rt.hipGraphDestroy(graph)
        hip.set_stream(old)
        outs.clear()
        del x, tgt, bias, act, pre, th, colsum, total, argmax, p, opt, params
        import gc
        gc.collect()
        _lib.check(l.zenu_hip_stream_destroy(stream), "stream_destroy")


def test_scheduled_adam_steps_through_graph_replays(hip):
    """`Adam::update` advances its step on every call (adam.rs:21-25).  A recorded update whose step is a
    kernel argument replays ONE step for ever; the scheduled update reads 1 - beta^t from a table in
    device memory and advances a device cursor, so replay i of one recorded update is step i.  Five
    consecutive eager AdamW steps with changing gradients, then the same five as replays of one graph:
    parameters and both moments equal bit for bit after every step; past the end of the table an
    update changes nothing and is counted."""
    from zenu_amd import _lib
    rt = _hip_runtime()
    l = hip.lib()
    M = hip.Matrix
    stream = C.c_void_p()
    _lib.check(l.zenu_hip_stream_create(C.byref(stream)), "stream_create")
    old = hip.get_stream()
    hip.set_stream(stream)
    graph, gexec = C.c_void_p(), C.c_void_p()
    opt = None
    try:
        r = np.random.default_rng(77)
        shapes = {"w1": (300, 257), "b1": (257,), "w2": (1 << 18,)}
        p0 = {k: (r.standard_normal(s) * 0.02).astype(np.float32) for k, s in shapes.items()}
        grads = [{k: (r.standard_normal(s) * (10.0 ** -i)).astype(np.float32) for k, s in shapes.items()} for i in range(9)]
        P = {k: M.from_numpy(v) for k, v in p0.items()}
        G = {k: M.alloc(s) for k, s in shapes.items()}
        params = {k: (P[k], G[k]) for k in shapes}

        def set_grads(i):
            for k in shapes:
                _lib.check(l.zenu_hip_memcpy_h2d(G[k].as_ptr(), grads[i][k].ctypes.data, grads[i][k].nbytes, stream), "h2d")

        def snapshot(o):
            hip.synchronize()
            return [t.to_numpy().copy() for k in shapes for t in (P[k], o.m[k], o.v[k])]

        eager = []
        ref = hip.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, params, ["w1", "w2"])
        for i in range(5):
            set_grads(i)
            ref.update(params)
            eager.append(snapshot(ref))

        for k in shapes:                                  # start again
            _lib.check(l.zenu_hip_memcpy_h2d(P[k].as_ptr(), p0[k].ctypes.data, p0[k].nbytes, stream), "h2d")
        opt = hip.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, params, ["w1", "w2"])
        opt.use_schedule(8)
        assert opt.schedule_state() == (1, 8, 0)
        hip.synchronize()
        assert rt.hipStreamBeginCapture(stream, 2) == 0
        try:
            opt.update(params)                            # recorded, not executed
        finally:
            rc = rt.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0
        assert rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        assert opt.schedule_state() == (1, 8, 0)          # recording advanced nothing
        for i in range(5):
            set_grads(i)
            assert rt.hipGraphLaunch(gexec, stream) == 0
            got = snapshot(opt)
            for a, b in zip(got, eager[i]):
                assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), ("replay", i)
            (P["w1"] + P["w1"]).sum(0)                    # eager work between the replays
        assert opt.schedule_state() == (6, 3, 0)
        # an eager (not recorded) scheduled call is the next step as well
        set_grads(5)
        opt.update(params)                                # step 6 through the schedule
        after6 = snapshot(opt)
        names = list(shapes)
        for j, k in enumerate(names):                     # the same step with the step number as a kernel argument
            _lib.check(l.zenu_hip_memcpy_h2d(P[k].as_ptr(), eager[4][3 * j].ctypes.data, p0[k].nbytes, stream), "h2d")
        ref2 = hip.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, params, ["w1", "w2"])
        for j, k in enumerate(names):
            _lib.check(l.zenu_hip_memcpy_h2d(ref2.m[k].as_ptr(), eager[4][3 * j + 1].ctypes.data, p0[k].nbytes, stream), "h2d")
            _lib.check(l.zenu_hip_memcpy_h2d(ref2.v[k].as_ptr(), eager[4][3 * j + 2].ctypes.data, p0[k].nbytes, stream), "h2d")
        ref2.step = 5
        ref2.update(params)
        for a, b in zip(after6, snapshot(ref2)):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), "eager scheduled step 6"
        for j, k in enumerate(names):                     # opt's parameters again
            _lib.check(l.zenu_hip_memcpy_h2d(P[k].as_ptr(), after6[3 * j].ctypes.data, p0[k].nbytes, stream), "h2d")
        # steps 7 and 8 exist; a ninth changes nothing and is counted
        for i in (6, 7):
            set_grads(i)
            assert rt.hipGraphLaunch(gexec, stream) == 0
        assert opt.schedule_state() == (9, 0, 0)
        before = snapshot(opt)
        set_grads(8)
        assert rt.hipGraphLaunch(gexec, stream) == 0
        for a, b in zip(snapshot(opt), before):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
        assert opt.schedule_state() == (9, 0, 1)
    finally:
        hip.synchronize()
        if gexec:
            rt.hipGraphExecDestroy(gexec)
        if graph:
            rt.hipGraphDestroy(graph)
        if opt is not None:
            opt.drop_schedule()
        hip.set_stream(old)
        P = G = params = ref = ref2 = opt = None   # freed before their stream goes
        import gc
        gc.collect()
        _lib.check(l.zenu_hip_stream_destroy(stream), "stream_destroy")


_POOL_OFF_CAPTURE = r"""
import ctypes as C, sys
import numpy as np
sys.path.insert(0, sys.argv[1])
import zenu_amd
from zenu_amd import _lib
rt = C.CDLL("libamdhip64.so")
vp = C.c_void_p
rt.hipStreamBeginCapture.argtypes = [vp, C.c_int]
rt.hipStreamEndCapture.argtypes = [vp, C.POINTER(vp)]
rt.hipGraphDestroy.argtypes = [vp]
l = zenu_amd.lib()
_lib.check(l.zenu_hip_init(0), "init")
stream = vp()
_lib.check(l.zenu_hip_stream_create(C.byref(stream)), "stream_create")
M = zenu_amd.Matrix
a = M.from_numpy(np.ones((4096, 256), dtype=np.float32))
out = M.alloc((256,))
p = vp()
_lib.check(l.zenu_hip_malloc(C.byref(p), 1 << 20, stream), "eager malloc with the pool off")
_lib.check(l.zenu_hip_sum_axis(_lib.F32, C.byref(out.desc()), C.byref(a.desc()), 0, stream), "eager split reduction")
assert rt.hipStreamBeginCapture(stream, 2) == 0
q = vp()
rc_malloc = l.zenu_hip_malloc(C.byref(q), 1 << 20, stream)
rc_free = l.zenu_hip_free(p, stream)
rc_reduce = l.zenu_hip_sum_axis(_lib.F32, C.byref(out.desc()), C.byref(a.desc()), 0, stream)   # needs partials
graph = vp()
rc_end = rt.hipStreamEndCapture(stream, C.byref(graph))
print("RC", rc_malloc, rc_free, rc_reduce, rc_end, bool(q.value))
if graph.value:
    rt.hipGraphDestroy(graph)
_lib.check(l.zenu_hip_free(p, stream), "free after the capture")
_lib.check(l.zenu_hip_sum_axis(_lib.F32, C.byref(out.desc()), C.byref(a.desc()), 0, stream), "reduction after the capture")
_lib.check(l.zenu_hip_stream_synchronize(stream), "sync")
assert np.array_equal(out.to_numpy(), np.full(256, 4096.0, dtype=np.float32))
print("DONE")
"""


def test_pool_off_refuses_scratch_while_capturing():
    """ZENU_USE_MEMPOOL=0: a capturing stream gets ZENU_ERR_UNSUPPORTED from the allocator and from a
    reduction that needs partials, before anything is recorded; the capture ends cleanly (no replay
    is needed to see that) and the same calls work again afterwards."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, ZENU_USE_MEMPOOL="0")
    r = subprocess.run([sys.executable, "-c", _POOL_OFF_CAPTURE, root], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, r.stdout + r.stderr
    line = [ln for ln in r.stdout.splitlines() if ln.startswith("RC")][0].split()
    from zenu_amd import _lib
    unsupported = str(_lib.ERR_UNSUPPORTED)
    assert line[1:4] == [unsupported] * 3, line
    assert line[4] == "0" and line[5] == "False", line
    assert "DONE" in r.stdout
