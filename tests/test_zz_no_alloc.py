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


def test_zz_no_ordinary_reduction_fell_back(hip):
    """Runs last: apart from the launches that tests/test_hip_parity.py forced onto that path (spin limit
    0), no split reduction of this process gave up polling for its partial results."""
    import ctypes as C
    from zenu_amd import _lib
    n = C.c_uint64()
    _lib.check(hip.lib().zenu_hip_reduce_fallback_count(C.byref(n)), "fallback count")
    assert n.value == getattr(hip, "_forced_fallbacks", 0)
