"""zenu_hip_sum_axis_noalloc: the allocation-free variant of zenu_hip_sum_axis.

Called through the C ABI and compared bit for bit with zenu_hip_sum_axis (same kernels, same launch
geometry, only the cross-workgroup scratch comes from the library's static device array instead of
the caching pool), on calls in a row that shrink (the static array keeps the previous call's
partials and must not leak them), in f32 and f64, for column, row and whole-row-split reductions, a
strided destination, and the documented refusals.  The pool's counters prove that the call takes
nothing from it; the sums themselves are checked against the CPU oracle to the bar of every sum here
(test_hip_parity.assert_sum_close: 1e-5 / 1e-12 relative).
"""
import ctypes as C

import numpy as np
import pytest

import zenu_oracle as zo
from test_hip_parity import assert_sum_close, bits_equal

pytestmark = pytest.mark.gpu


def _stats(hip):
    from zenu_amd import _lib
    st = _lib.MempoolStats()
    _lib.check(hip.lib().zenu_hip_mempool_stats(C.byref(st)), "stats")
    return st


def _both(hip, X, axis, out_shape, dt):
    """(noalloc result, zenu_hip_sum_axis result), the first produced without touching the pool"""
    from zenu_amd import _lib
    l = hip.lib()
    M = hip.Matrix
    a, b = M.alloc(out_shape, dtype=dt), M.alloc(out_shape, dtype=dt)
    code = _lib.F32 if np.dtype(dt) == np.float32 else _lib.F64
    before = _stats(hip)
    rc = l.zenu_hip_sum_axis_noalloc(code, C.byref(a.desc()), C.byref(X.desc()), axis, hip.get_stream())
    after = _stats(hip)
    assert rc == _lib.OK, rc
    assert after.n_alloc_calls == before.n_alloc_calls and after.n_driver_allocs == before.n_driver_allocs
    _lib.check(l.zenu_hip_sum_axis(code, C.byref(b.desc()), C.byref(X.desc()), axis, hip.get_stream()), "sum_axis")
    return a.to_numpy(), b.to_numpy()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_sum_axis_noalloc_matches_sum_axis(hip, dt):
    r = np.random.default_rng(5)
    # in a row, shrinking: column reduction split over workgroups; a smaller ragged one; rows split
    # with the counter tree (4 outputs x 128 splits); rows split flat; unsplit; a single output
    cases = [((4096, 2048), 0), ((1000, 516), 0), ((4, 1 << 20), 1), ((40, 50000), 1), ((3000, 700), 1),
             ((1 << 21,), 0), ((257, 3, 130), 0), ((6, 900, 64), 1), ((5, 7), 0)]
    for shape, axis in cases:
        x = r.standard_normal(shape).astype(dt)
        X = hip.Matrix.from_numpy(x)
        oshape = shape[:axis] + shape[axis + 1:]
        got, ref = _both(hip, X, axis, oshape, dt)
        assert bits_equal(got, ref), (shape, axis)
        # against the CPU oracle and the exact f64 sum, with the rule every sum test here uses
        assert_sum_close(got, zo.sum_axis(x, axis), x, axis, f"{shape} axis {axis}", cpu_slack=shape[axis] > 8192)
        del X


def test_sum_axis_noalloc_views_and_limits(hip):
    from zenu_amd import _lib
    l = hip.lib()
    M = hip.Matrix
    r = np.random.default_rng(6)
    x = r.standard_normal((2048, 1024)).astype(np.float32)
    X = M.from_numpy(x)
    s = hip.get_stream()
    # a transposed source is reduced in place; keep_dim destination
    got, ref = _both(hip, X.transpose(), 0, (1, 2048), np.float32)
    assert np.array_equal(got, ref)
    # strided destination: every second element of a longer vector, staged through the static array
    D = M.from_numpy(np.full(2048, -7.0, dtype=np.float32))
    dview = D.slice(slice(0, 2048, 2))
    before = _stats(hip)
    rc = l.zenu_hip_sum_axis_noalloc(_lib.F32, C.byref(dview.desc()), C.byref(X.desc()), 0, s)
    assert rc == _lib.OK and _stats(hip).n_alloc_calls == before.n_alloc_calls
    E = M.alloc((1024,))
    _lib.check(l.zenu_hip_sum_axis(_lib.F32, C.byref(E.desc()), C.byref(X.desc()), 0, s), "sum_axis")
    d = D.to_numpy()
    assert np.array_equal(d[0::2], E.to_numpy()) and np.all(d[1::2] == -7.0)
    # refusals, each with nothing launched: a source that needs a staging copy ...
    g = M.from_numpy(r.standard_normal((64, 64, 8)).astype(np.float32))
    gv = g.slice(slice(None), slice(0, 64, 2), slice(0, 8, 2))      # kept dims: neither one stride chain nor a unit-stride run
    o = M.from_numpy(np.full((32, 4), 3.0, dtype=np.float32))
    assert l.zenu_hip_sum_axis_noalloc(_lib.F32, C.byref(o.desc()), C.byref(gv.desc()), 0, s) == _lib.ERR_UNSUPPORTED
    # ... a strided destination larger than the staging area (512 KiB) ...
    big = M.alloc((300000, 2))
    bview = big.slice(slice(None), slice(0, 1))                      # 300000 x 1, stride 2
    src2 = M.alloc((2, 300000, 1))
    assert l.zenu_hip_sum_axis_noalloc(_lib.F32, C.byref(bview.desc()), C.byref(src2.desc()), 0, s) == _lib.ERR_SCRATCH_LIMIT
    # ... and the ordinary shape / axis errors
    assert l.zenu_hip_sum_axis_noalloc(_lib.F32, C.byref(o.desc()), C.byref(X.desc()), 0, s) == _lib.ERR_SHAPE
    assert l.zenu_hip_sum_axis_noalloc(_lib.F32, C.byref(o.desc()), C.byref(X.desc()), 5, s) == _lib.ERR_AXIS
    hip.synchronize()
    assert np.all(o.to_numpy() == 3.0)
    assert b"static scratch" in l.zenu_hip_status_string(_lib.ERR_SCRATCH_LIMIT)
    del big, bview, src2


def test_noalloc_large_split_then_small_split_reuses_the_same_scratch(hip):
    """A large split reduction fills the static partials; the small one after it uses the first bytes of
    the same area with fewer splits and different data: nothing of the large call's partials may
    reach the small call's result (and the other way round on the third call)."""
    r = np.random.default_rng(9)
    big = (r.standard_normal((8192, 1024)) * 1000).astype(np.float32)      # 16 splits x 1024 outputs
    small = r.standard_normal((520, 256)).astype(np.float32)                # fewer splits, fewer outputs
    B, S = hip.Matrix.from_numpy(big), hip.Matrix.from_numpy(small)
    for X, x in ((B, big), (S, small), (B, big), (S, small)):
        got, ref = _both(hip, X, 0, (x.shape[1],), np.float32)
        assert bits_equal(got, ref), x.shape
        assert_sum_close(got, zo.sum_axis(x, 0), x, 0, f"{x.shape} axis 0")


def test_noalloc_call_recorded_into_a_graph(hip):
    """The call is meant for code under HIP-graph capture: record it (a split column reduction and a split
    row reduction, with their counter fills) into a graph, replay the graph on new inputs with eager
    reductions on the same stream in between, and compare every replay bit for bit with
    zenu_hip_sum_axis on the same inputs.  The pool's counters do not move during the capture."""
    from zenu_amd import _lib
    from test_hip_graph import _hip_runtime
    rt = _hip_runtime()
    l = hip.lib()
    M = hip.Matrix
    stream = C.c_void_p()
    _lib.check(l.zenu_hip_stream_create(C.byref(stream)), "stream_create")
    old = hip.get_stream()
    hip.set_stream(stream)
    graph, gexec = C.c_void_p(), C.c_void_p()
    try:
        r = np.random.default_rng(10)
        inputs = [r.standard_normal((4096, 512)).astype(np.float32) * s for s in (1.0, 3.0, 0.25)]
        X = M.from_numpy(inputs[0])
        Xr = X.reshape((4, 4096 * 128))
        cols, rows = M.alloc((512,)), M.alloc((4,))
        ecols, erows = M.alloc((512,)), M.alloc((4,))

        def sequence(fn, oc, orow):
            _lib.check(fn(_lib.F32, C.byref(oc.desc()), C.byref(X.desc()), 0, stream), "cols")
            _lib.check(fn(_lib.F32, C.byref(orow.desc()), C.byref(Xr.desc()), 1, stream), "rows")

        sequence(l.zenu_hip_sum_axis_noalloc, cols, rows)                 # eager once
        hip.synchronize()
        before = _stats(hip)
        assert rt.hipStreamBeginCapture(stream, 2) == 0
        try:
            sequence(l.zenu_hip_sum_axis_noalloc, cols, rows)
        finally:
            rc = rt.hipStreamEndCapture(stream, C.byref(graph))
        assert rc == 0
        after = _stats(hip)
        assert after.n_alloc_calls == before.n_alloc_calls and after.n_driver_allocs == before.n_driver_allocs
        assert rt.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
        for i, inp in enumerate(inputs + inputs[:1]):
            _lib.check(l.zenu_hip_memcpy_h2d(X.as_ptr(), inp.ctypes.data, inp.nbytes, stream), "h2d")
            _lib.check(l.zenu_hip_memset_zero(cols.as_ptr(), 512 * 4, stream), "zero")
            _lib.check(l.zenu_hip_memset_zero(rows.as_ptr(), 4 * 4, stream), "zero")
            assert rt.hipGraphLaunch(gexec, stream) == 0
            hip.synchronize()
            got = cols.to_numpy().copy(), rows.to_numpy().copy()
            sequence(l.zenu_hip_sum_axis, ecols, erows)                   # eager work between the replays
            hip.synchronize()
            assert bits_equal(got[0], ecols.to_numpy()) and bits_equal(got[1], erows.to_numpy()), i
            assert_sum_close(got[0], zo.sum_axis(inp, 0), inp, 0, "replayed column sums")
    finally:
        hip.synchronize()
        if gexec:
            rt.hipGraphExecDestroy(gexec)
        if graph:
            rt.hipGraphDestroy(graph)
        hip.set_stream(old)
        X = Xr = cols = rows = ecols = erows = None      # freed before their stream goes
        import gc
        gc.collect()
        _lib.check(l.zenu_hip_stream_destroy(stream), "stream_destroy")

def test_zz_no_ordinary_reduction_fell_back(hip):
    """Runs last: apart from the launches that tests/test_hip_parity.py forced onto that path (spin limit
    0), no split reduction of this process gave up polling for its partial results."""
    import ctypes as C
    from zenu_amd import _lib
    n = C.c_uint64()
    _lib.check(hip.lib().zenu_hip_reduce_fallback_count(C.byref(n)), "fallback count")
    assert n.value == getattr(hip, "_forced_fallbacks", 0)
