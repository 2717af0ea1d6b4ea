"""Fused classifier-head entry points (softmax, softmax backward, cross-entropy forward and backward,
bias add + ReLU, ReLU backward, clip) against the op-by-op chains on the CPU oracle
(tests/cpu_matrix.py restates each chain with the reference's file:line).

Bars: everything is bit-exact in f32 wherever the chain's own summation order is the fused kernel's
(one thread per softmax line: reduced length <= 64 or an inner stride), since exp and log (f32 and f64)
restate the host libm; tree sums rel 1e-5 f32 / 1e-12 f64.
"""
import ctypes as C

import numpy as np
import pytest

import cpu_matrix
from cpu_matrix import CpuMatrix

pytestmark = pytest.mark.gpu


def bits_equal(a, b):
    a = np.ascontiguousarray(a).reshape(-1)
    b = np.ascontiguousarray(b).reshape(-1)
    ui = np.uint32 if a.dtype == np.float32 else np.uint64
    return a.shape == b.shape and np.array_equal(a.view(ui), b.view(ui))


def rel_err(got, ref):
    got = got.astype(np.float64)
    ref = ref.astype(np.float64)
    return float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1e-300)))


SOFTMAX_SHAPES = [
    # shape, axis
    ((256, 10), 1),        # configs[4] logits: one thread per row, index-order sum
    ((7, 64), 1),
    ((64, 1000), 1),       # workgroup per row, row in registers (vector loads)
    ((33, 1027), 1),       # not a multiple of the vector width
    ((5, 5000), 1),        # three-pass rows (f32: > 4096)
    ((3, 9001), 1),
    ((100, 37), 0),        # reduced axis first: one thread per column
    ((4, 50, 6), 1),       # middle axis
    ((2, 3, 4, 5), 3),
    ((17,), 0),
]


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("shape,axis", SOFTMAX_SHAPES, ids=lambda v: str(v))
def test_softmax_forward_backward(hip, dtype, shape, axis):
    print(f"[case] softmax {shape} axis {axis} {np.dtype(dtype).name}", flush=True)
    r = np.random.default_rng(abs(hash((shape, axis))) % 2**31)
    x = (r.standard_normal(shape) * 3).astype(dtype)
    gy = r.standard_normal(shape).astype(dtype)
    R = shape[axis]
    inner = int(np.prod(shape[axis + 1:]))
    in_order = R <= 64 or inner > 1     # one thread per line: the chain's own summation order
    # exp within 2 ulp when the denominators are summed alike; otherwise the sum bar applies
    if in_order:
        tol = 2e-6 if dtype == np.float32 else 1e-14
    else:
        tol = 1e-5 if dtype == np.float32 else 1e-12

    ref = CpuMatrix.zeros(shape, dtype)
    ref.softmax_assign(CpuMatrix.from_numpy(x), axis)
    out = hip.Matrix.zeros(shape, dtype)
    out.softmax_assign(hip.Matrix.from_numpy(x), axis)
    y = out.to_numpy()
    assert rel_err(y, ref.a) <= tol
    if in_order:
        assert bits_equal(y, ref.a)         # exp is the host libm's algorithm and the sums run in index order
    assert np.allclose(y.sum(axis=axis, dtype=np.float64), 1.0, atol=1e-5 if dtype == np.float32 else 1e-12)

    # in place (to == src)
    inpl = hip.Matrix.from_numpy(x)
    inpl.softmax_assign(inpl, axis)
    assert bits_equal(inpl.to_numpy(), y)

    # backward from the SAME y on both devices: arithmetic only
    gref = cpu_matrix.softmax_backward(CpuMatrix.from_numpy(y), CpuMatrix.from_numpy(gy), axis).a
    g = hip.softmax_backward(hip.Matrix.from_numpy(y), hip.Matrix.from_numpy(gy), axis).to_numpy()
    if in_order:
        assert bits_equal(g, gref)          # index-order sum on both sides
    else:
        scale = np.max(np.abs(gref))
        assert np.max(np.abs(g.astype(np.float64) - gref)) <= (1e-5 if dtype == np.float32 else 1e-12) * scale


@pytest.mark.parametrize("seed", range(4))
def test_fused_fuzz(hip, seed):
    """seeded random shapes (1-4 dims, the softmax axis 1 .. 1500 long), random axis, f32 / f64:
    softmax and its backward against the op-by-op chains with the bars of test_softmax_forward_backward,
    bias add + ReLU (bit-exact), and for 2-d shapes the cross-entropy loss and its backward"""
    r = np.random.default_rng(900 + seed)
    for case in range(25):
        dtype = np.float32 if r.random() < 0.6 else np.float64
        nd = int(r.integers(1, 5))
        axis = int(r.integers(0, nd))
        shape = tuple(int(r.integers(1, 1500)) if d == axis and r.random() < 0.6 else int(r.integers(1, 9)) for d in range(nd))
        print(f"[fuzz] seed {seed} case {case}: {shape} axis {axis} {np.dtype(dtype).name}", flush=True)
        x = (r.standard_normal(shape) * 3).astype(dtype)
        gy = r.standard_normal(shape).astype(dtype)
        R, inner = shape[axis], int(np.prod(shape[axis + 1:]))
        in_order = R <= 64 or inner > 1
        tol = (2e-6 if dtype == np.float32 else 1e-14) if in_order else (1e-5 if dtype == np.float32 else 1e-12)
        ref = CpuMatrix.zeros(shape, dtype)
        ref.softmax_assign(CpuMatrix.from_numpy(x), axis)
        out = hip.Matrix.zeros(shape, dtype)
        out.softmax_assign(hip.Matrix.from_numpy(x), axis)
        y = out.to_numpy()
        assert rel_err(y, ref.a) <= tol
        if in_order:
            assert bits_equal(y, ref.a)
        gref = cpu_matrix.softmax_backward(CpuMatrix.from_numpy(y), CpuMatrix.from_numpy(gy), axis).a
        g = hip.softmax_backward(hip.Matrix.from_numpy(y), hip.Matrix.from_numpy(gy), axis).to_numpy()
        if in_order:
            assert bits_equal(g, gref)
        else:
            assert np.max(np.abs(g.astype(np.float64) - gref)) <= (1e-5 if dtype == np.float32 else 1e-12) * max(np.max(np.abs(gref)), 1e-30)
        if nd >= 2:
            # bias over the last dim, added and rectified: arithmetic only, bit-exact
            bias = r.standard_normal(shape[-1]).astype(dtype)
            alpha = float(r.choice([0.0, 0.2]))
            cref = CpuMatrix.zeros(shape, dtype)
            cpre = CpuMatrix.zeros(shape, dtype)
            cref.bias_add_relu(CpuMatrix.from_numpy(x), CpuMatrix.from_numpy(bias), alpha, cpre)
            act, pre = hip.Matrix.zeros(shape, dtype), hip.Matrix.zeros(shape, dtype)
            act.bias_add_relu(hip.Matrix.from_numpy(x), hip.Matrix.from_numpy(bias), alpha, pre)
            assert bits_equal(act.to_numpy(), cref.a) and bits_equal(pre.to_numpy(), cpre.a)


def test_softmax_strided_views(hip):
    """transposed source and sliced destination go through contiguous staging"""
    r = np.random.default_rng(5)
    x = r.standard_normal((40, 24)).astype(np.float32)
    ref = CpuMatrix.zeros((24, 40))
    ref.softmax_assign(CpuMatrix.from_numpy(x).transpose(), 1)
    big = hip.Matrix.zeros((24, 80))
    dst = big.slice(slice(None), slice(0, 80, 2))
    dst.softmax_assign(hip.Matrix.from_numpy(x).transpose(), 1)
    assert rel_err(big.to_numpy()[:, ::2], ref.a) <= 2e-6
    assert np.all(big.to_numpy()[:, 1::2] == 0)


def test_softmax_rows_divide_like_the_chain(hip):
    """The workgroup-per-row kernel adds the row in a tree, so its sum S may differ from the chain's
    index-order sum by a few units in the last place -- but every element of a row must be the
    correctly rounded exp(x - max) / S for ONE such S, as the chain's element-wise division would
    give.  Rows: random
    logits of several spreads, spreads that put elements below 2^-80 and at zero, -inf entries, equal
    entries (S a power of two), lengths on both sides of the row-in-registers limit."""
    import zenu_oracle as zo
    r = np.random.default_rng(11)
    for R in (4096, 1000, 5000):
        rows = [r.standard_normal(R) * s for s in (0.1, 1.0, 3.0, 10.0, 30.0)]
        rows.append(np.linspace(-120.0, 0.0, R))                       # tiny, subnormal and zero quotients
        rows.append(np.where(r.random(R) < 0.3, -np.inf, r.standard_normal(R)))
        rows.append(np.full(R, 0.25))
        rows += [r.standard_normal(R) * 2.0 for _ in range(24)]
        x = np.ascontiguousarray(np.array(rows, dtype=np.float32))
        out = hip.Matrix.zeros(x.shape)
        out.softmax_assign(hip.Matrix.from_numpy(x), 1)
        got = out.to_numpy()
        m = x.max(axis=1, keepdims=True)
        a = np.empty_like(x)
        zo.unary(zo.EXP, a, np.ascontiguousarray(x - m))               # the chain's exp, bit-exact on the device
        for i in range(x.shape[0]):
            s0 = np.float32(a[i].astype(np.float64).sum())             # the exact sum, rounded: any summation order lands near it
            cand = s0
            for _ in range(64):
                cand = np.nextafter(cand, np.float32(0))
            matched = False
            for _ in range(129):
                with np.errstate(all="ignore"):
                    if bits_equal(got[i], (a[i] / cand).astype(np.float32)):
                        matched = True
                        break
                cand = np.nextafter(cand, np.float32(np.inf))
            assert matched, f"R={R} row {i}: no single divisor near {s0!r} reproduces the row"


def test_softmax_special_rows(hip):
    """NaN in position 0 / elsewhere and an all -inf row poison the row exactly as in the chain; a row
    with +inf gives NaN at the inf (inf - inf) and 0 elsewhere... all NaN after the division"""
    x = np.array([[np.nan, 1, 2, 3], [1, np.nan, 2, 3], [-np.inf] * 4, [1, np.inf, 2, 3], [5, 5, 5, 5]],
                 dtype=np.float32)
    ref = CpuMatrix.zeros(x.shape)
    ref.softmax_assign(CpuMatrix.from_numpy(x), 1)
    out = hip.Matrix.zeros(x.shape)
    out.softmax_assign(hip.Matrix.from_numpy(x), 1)
    got = out.to_numpy()
    assert np.array_equal(np.isnan(got), np.isnan(ref.a))
    assert bits_equal(got[4], ref.a[4])


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("n,c", [(256, 10), (1, 4), (255, 13), (7, 1), (128, 16), (3, 2), (1000, 64), (50, 1000), (70000, 3)])
def test_cross_entropy(hip, dtype, n, c):
    print(f"[case] cross_entropy {n}x{c} {np.dtype(dtype).name}", flush=True)
    r = np.random.default_rng(n * 131 + c)
    pred = r.standard_normal((n, c)).astype(dtype)
    ans = np.zeros((n, c), dtype=dtype)
    ans[np.arange(n), r.integers(0, c, n)] = 1
    sum_tol = 1e-5 if dtype == np.float32 else 1e-12
    tol = (2e-6 if dtype == np.float32 else 1e-14) if c <= 64 else sum_tol

    loss_ref, prob_ref = cpu_matrix.cross_entropy(CpuMatrix.from_numpy(pred), CpuMatrix.from_numpy(ans))
    loss, prob = hip.cross_entropy(hip.Matrix.from_numpy(pred), hip.Matrix.from_numpy(ans))
    assert rel_err(prob.to_numpy(), prob_ref.a) <= tol
    if c <= 64:
        assert bits_equal(prob.to_numpy(), prob_ref.a)
    exact = -np.sum(ans.astype(np.float64) * np.log(prob_ref.a.astype(np.float64))) / n
    assert abs(float(loss.to_numpy()) - exact) <= sum_tol * abs(exact)
    assert abs(float(loss.to_numpy()) - float(loss_ref.a)) <= 4 * sum_tol * abs(exact)

    # backward from the same softmax output on both devices
    p = prob.to_numpy()
    gref = cpu_matrix.cross_entropy_backward(CpuMatrix.from_numpy(p), CpuMatrix.from_numpy(ans)).a
    g = hip.cross_entropy_backward(hip.Matrix.from_numpy(p), hip.Matrix.from_numpy(ans)).to_numpy()
    if c <= 64:
        assert bits_equal(g, gref)
    else:
        assert np.max(np.abs(g.astype(np.float64) - gref)) <= sum_tol * np.max(np.abs(gref))
    # closed form: (softmax - onehot) / N
    closed = (p.astype(np.float64) - ans) / n
    assert np.max(np.abs(g - closed)) <= 1e-6 / n * 4 + (1e-6 if dtype == np.float32 else 1e-14)

    # a gradient arriving at the loss scales the result
    gl = np.array(-2.5, dtype=dtype)
    gref2 = cpu_matrix.cross_entropy_backward(CpuMatrix.from_numpy(p), CpuMatrix.from_numpy(ans),
                                              CpuMatrix.from_numpy(gl)).a
    g2 = hip.cross_entropy_backward(hip.Matrix.from_numpy(p), hip.Matrix.from_numpy(ans),
                                    hip.Matrix.from_numpy(gl)).to_numpy()
    if c <= 64:
        assert bits_equal(g2, gref2)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("shape", [(256, 512), (3, 5, 7), (1000, 10), (4096, 4096)])
@pytest.mark.parametrize("alpha", [0.0, 0.2])
def test_bias_add_relu_and_backward(hip, dtype, shape, alpha):
    print(f"[case] bias_add_relu {shape} {np.dtype(dtype).name} alpha {alpha}", flush=True)
    r = np.random.default_rng(shape[0])
    z = r.standard_normal(shape).astype(dtype)
    z.reshape(-1)[::17] = 0.0
    z.reshape(-1)[5::29] = -0.0
    b = r.standard_normal(shape[-1]).astype(dtype)
    b[::3] = 0.0
    gy = r.standard_normal(shape).astype(dtype)

    pre_ref, act_ref = CpuMatrix.zeros(shape, dtype), CpuMatrix.zeros(shape, dtype)
    act_ref.bias_add_relu(CpuMatrix.from_numpy(z), CpuMatrix.from_numpy(b), alpha, pre=pre_ref)
    pre, act = hip.Matrix.zeros(shape, dtype), hip.Matrix.zeros(shape, dtype)
    act.bias_add_relu(hip.Matrix.from_numpy(z), hip.Matrix.from_numpy(b), alpha, pre=pre)
    assert bits_equal(pre.to_numpy(), pre_ref.a)
    assert bits_equal(act.to_numpy(), act_ref.a)      # includes the -0.0 of alpha*x for alpha = 0
    act2 = hip.Matrix.zeros(shape, dtype)
    act2.bias_add_relu(hip.Matrix.from_numpy(z), hip.Matrix.from_numpy(b), alpha)
    assert bits_equal(act2.to_numpy(), act_ref.a)

    gref = CpuMatrix.zeros(shape, dtype)
    gref.relu_backward(CpuMatrix.from_numpy(gy), pre_ref, alpha)
    g = hip.Matrix.zeros(shape, dtype)
    g.relu_backward(hip.Matrix.from_numpy(gy), pre, alpha)
    assert bits_equal(g.to_numpy(), gref.a)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_clip_parity(hip, dtype):
    r = np.random.default_rng(11)
    x = (r.standard_normal((257, 129)) * 2).astype(dtype)
    x[0, :4] = [np.nan, np.inf, -np.inf, -0.0]
    x[1, :2] = [-1.0, 1.5]                     # exactly on the bounds
    cx, hx = CpuMatrix.from_numpy(x), hip.Matrix.from_numpy(x)
    assert bits_equal(hx.clip(-1.0, 1.5).to_numpy(), cx.clip(-1.0, 1.5).a)
    assert bits_equal(hx.clip_backward_mask(-1.0, 1.5).to_numpy(), cx.clip_backward_mask(-1.0, 1.5).a)
    # strided views, same strides on both operands (the reference indexes the mask with the
    # input's stride, clip.rs:90-96, so only equal strides are well defined there)
    cv, hv = cx.slice(slice(None), slice(0, 129, 2)), hx.slice(slice(None), slice(0, 129, 2))
    cv.clip_assign(-0.5, 0.5)
    hv.clip_assign(-0.5, 0.5)
    assert bits_equal(hx.to_numpy(), cx.a)
    cv.clip_backward_assign_mask(-0.25, 0.25)
    hv.clip_backward_assign_mask(-0.25, 0.25)
    assert bits_equal(hx.to_numpy(), cx.a)


def test_reference_named_clip_and_conv_bias_add(hip):
    """array_clip_* / conv_bias_add_* keep the reference's names and argument order
    (zenu-cuda-kernel-sys/kernel/array_scalar.h:97-106, array_array.h:27-28)"""
    L = hip.lib()
    fp = C.POINTER(C.c_float)
    a = np.arange(6, dtype=np.float32)
    d = hip.Matrix.from_numpy(a)
    o = hip.Matrix.zeros([6])
    L.array_clip_float.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_float, C.c_float]
    L.array_clip_float.restype = None
    L.array_clip_float(d.as_ptr(), o.as_ptr(), 6, 1, 1, 1.0, 2.0)
    assert np.array_equal(o.to_numpy(), [1, 1, 2, 2, 2, 2])
    L.array_clip_backward_float.argtypes = [C.c_void_p, C.c_void_p, C.c_float, C.c_float, C.c_int, C.c_int, C.c_int]
    L.array_clip_backward_float.restype = None
    L.array_clip_backward_float(d.as_ptr(), d.as_ptr(), 2.0, 1.0, 6, 1, 1)   # kernel/mod.rs:1316
    assert np.array_equal(d.to_numpy(), [0, 1, 1, 0, 0, 0])

    # conv_bias_add: [N, C, H*W] + bias[C], plus totals that end inside an image / a channel
    r = np.random.default_rng(3)
    n, c, hw = 3, 5, 14
    x = r.standard_normal(n * c * hw).astype(np.float64)
    bias = r.standard_normal(c).astype(np.float64)
    L.conv_bias_add_double.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int]
    L.conv_bias_add_double.restype = None
    for total in (n * c * hw, n * c * hw - hw, n * c * hw - 3, 9):
        dx, db = hip.Matrix.from_numpy(x), hip.Matrix.from_numpy(bias)
        out = hip.Matrix.zeros([n * c * hw], np.float64)
        L.conv_bias_add_double(dx.as_ptr(), out.as_ptr(), hw, db.as_ptr(), c, total)
        idx = np.arange(total)
        exp = np.zeros_like(x)
        exp[:total] = x[:total] + bias[(idx // hw) % c]
        assert bits_equal(out.to_numpy(), exp), total
    del fp


def test_conv2d_bias_add_and_backward(hip):
    """ConvBias (zenu-matrix/src/nn/conv/mod.rs:84-107, cpu/bias.rs): the forward add is bit-exact;
    the bias gradient is three sums (sum bar), and the reference-named entry
    conv2d_bias_bkwd_<type> (conv2d_bkwd_data.h:7-17) gives the same numbers."""
    r = np.random.default_rng(23)
    for dt, tol in ((np.float32, 1e-5), (np.float64, 1e-12)):
        for (n, c, h, w) in ((4, 3, 5, 7), (16, 64, 28, 28), (1, 8, 1, 1), (3, 1, 2, 33)):
            x = r.standard_normal((n, c, h, w)).astype(dt)
            b = r.standard_normal((1, c, 1, 1)).astype(dt)
            hx, hb, ho = hip.Matrix.from_numpy(x), hip.Matrix.from_numpy(b), hip.Matrix.zeros(x.shape, dt)
            cx, cb, co = CpuMatrix.from_numpy(x), CpuMatrix.from_numpy(b), CpuMatrix.zeros(x.shape, dt)
            hip.conv2d_bias_add(hx, hb, ho)
            cpu_matrix.conv2d_bias_add(cx, cb, co)
            assert bits_equal(ho.to_numpy(), co.a)
            hg, cg = hip.Matrix.zeros(b.shape, dt), CpuMatrix.zeros(b.shape, dt)
            hip.conv2d_bias_bkwd(hx, hg)
            cpu_matrix.conv2d_bias_bkwd(cx, cg)
            scale = np.maximum(np.abs(cg.a), np.abs(x).sum(axis=(0, 2, 3)).reshape(b.shape) / np.sqrt(n * h * w))
            assert np.all(np.abs(hg.to_numpy() - cg.a) <= tol * scale), (dt, n, c, h, w)
            # the reference-named C entry point
            L = hip.lib()
            f = getattr(L, "conv2d_bias_bkwd_" + ("float" if dt == np.float32 else "double"))
            f.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int]
            f.restype = None
            hg2 = hip.Matrix.zeros(b.shape, dt)
            f(hx.as_ptr(), hg2.as_ptr(), n, c, h, w)
            assert bits_equal(hg2.to_numpy(), hg.to_numpy())
    with pytest.raises(hip.ZenuHipError):
        hip.conv2d_bias_bkwd(hx, hip.Matrix.zeros((1, c + 1, 1, 1), dt))


def test_tanh_and_sigmoid_backward(hip):
    """One-pass backward of tanh (zenu-autograd/src/functions/tanh.rs:30-37) and of the sigmoid
    composite (activation/sigmoid.rs:7-15) against the op-by-op chains on the CPU: bit-exact in
    f32 and f64 (cosh is the host libm's algorithm in both).  Also strided views and the
    closed form d tanh = 1 - tanh^2, d sigmoid = s (1 - s)."""
    r = np.random.default_rng(29)
    x32 = np.concatenate([r.standard_normal(100000) * 3, r.uniform(-95, 95, 20000),
                          [0.0, -0.0, 1e-30, 22.0, -22.0, 88.0, 89.5, -89.5, 100.0, np.inf, -np.inf, np.nan]]).astype(np.float32)
    g32 = r.standard_normal(x32.size).astype(np.float32)
    for dt, bar in ((np.float32, 0), (np.float64, 0)):
        x, gy = x32.astype(dt), g32.astype(dt)
        hx, hg = hip.Matrix.from_numpy(x), hip.Matrix.from_numpy(gy)
        cx, cg = CpuMatrix.from_numpy(x), CpuMatrix.from_numpy(gy)
        for name in ("tanh_backward", "sigmoid_backward"):
            ho, co = hip.Matrix.zeros(x.shape, dt), CpuMatrix.zeros(x.shape, dt)
            getattr(ho, name)(hg, hx)
            with np.errstate(all="ignore"):
                getattr(co, name)(cg, cx)
            got, exp = ho.to_numpy(), co.a
            assert np.array_equal(np.isnan(got), np.isnan(exp)), (name, dt)
            ok = ~np.isnan(exp)
            if bar == 0:
                assert bits_equal(got[ok], exp[ok]), (name, dt)
            else:
                fin = ok & np.isfinite(exp) & (exp != 0)
                assert np.max(np.abs(got[fin] - exp[fin]) / np.abs(exp[fin])) <= bar * np.finfo(dt).eps, (name, dt)
    # closed forms, f64, moderate arguments
    x = r.standard_normal(50000) * 2
    one = np.ones_like(x)
    hx, h1 = hip.Matrix.from_numpy(x), hip.Matrix.from_numpy(one)
    o = hip.Matrix.zeros(x.shape, np.float64)
    o.tanh_backward(h1, hx)
    assert np.allclose(o.to_numpy(), 1 - np.tanh(x) ** 2, rtol=1e-13, atol=1e-15)
    o.sigmoid_backward(h1, hx)
    s = 1 / (1 + np.exp(-x))
    assert np.allclose(o.to_numpy(), s * (1 - s), rtol=1e-13, atol=1e-15)
    # strided views: transposed x, every other row of gy
    m = r.standard_normal((64, 96)).astype(np.float32)
    g = r.standard_normal((192, 64)).astype(np.float32)
    hm, hg = hip.Matrix.from_numpy(m).transpose(), hip.Matrix.from_numpy(g).slice(slice(None, None, 2))
    cm, cg = CpuMatrix.from_numpy(np.ascontiguousarray(m.T)), CpuMatrix.from_numpy(np.ascontiguousarray(g[::2]))
    ho, co = hip.Matrix.zeros((96, 64)), CpuMatrix.zeros((96, 64))
    ho.sigmoid_backward(hg, hm)
    co.sigmoid_backward(cg, cm)
    assert bits_equal(ho.to_numpy(), co.a)
    with pytest.raises(hip.ZenuHipError):
        ho.tanh_backward(hg, hip.Matrix.zeros((64, 96)))


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("shape", [(256, 512), (256, 10), (1000, 130), (3, 40, 64), (8192, 4096), (64, 18), (5000, 16)])
@pytest.mark.parametrize("alpha", [0.0, 0.2])
def test_relu_backward_bias_grad(hip, dtype, shape, alpha):
    """gx and the bias gradient in one pass: gx is the bits of relu_backward (and of the oracle's mask
    chain), the bias gradient the bits of sum_to over that gx when the gradient is 2-d (same kernel,
    same geometry) and within the bar of every sum against the oracle and the exact f64 sums; shapes
    on both sides of the one-launch conditions (column count below 16 or no multiple of the vector
    width, more than two dims)."""
    print(f"[case] relu_backward_bias_grad {shape} {np.dtype(dtype).name} alpha {alpha}", flush=True)
    r = np.random.default_rng(shape[0] + 7 * shape[-1])
    x = r.standard_normal(shape).astype(dtype)
    x.reshape(-1)[::13] = 0.0
    x.reshape(-1)[3::31] = -0.0
    gy = r.standard_normal(shape).astype(dtype)
    n = shape[-1]
    M = hip.Matrix
    X, GY = M.from_numpy(x), M.from_numpy(gy)
    gx, gb = M.alloc(shape, dtype), M.from_numpy(np.full(n, 77.0, dtype=dtype))
    gx.relu_backward_bias_grad(gb, GY, X, alpha)
    gx2 = M.alloc(shape, dtype)
    gx2.relu_backward(GY, X, alpha)
    assert bits_equal(gx.to_numpy(), gx2.to_numpy())
    gref, gbref = CpuMatrix.zeros(shape, dtype), CpuMatrix.zeros((n,), dtype)
    gref.relu_backward_bias_grad(gbref, CpuMatrix.from_numpy(gy), CpuMatrix.from_numpy(x), alpha)
    assert bits_equal(gx.to_numpy(), gref.a)
    if len(shape) == 2:
        gb2 = M.alloc((n,), dtype)
        hip.sum_to(gx2, gb2)
        assert bits_equal(gb.to_numpy(), gb2.to_numpy())
    g64 = gref.a.astype(np.float64).reshape(-1, n)
    exact = g64.sum(0)
    scale = np.maximum(np.abs(exact), np.abs(g64).sum(0) / np.sqrt(g64.shape[0]))
    tol = 1e-5 if dtype == np.float32 else 1e-12
    assert np.all(np.abs(gb.to_numpy() - exact) <= tol * scale)
    assert np.all(np.abs(gb.to_numpy() - gbref.a) <= 2 * tol * scale)
    # twice in a row: the same bits (fixed merge order), and in place (gx == gy)
    gb3 = M.alloc((n,), dtype)
    GY.relu_backward_bias_grad(gb3, GY, X, alpha)
    assert bits_equal(GY.to_numpy(), gx.to_numpy()) and bits_equal(gb3.to_numpy(), gb.to_numpy())


def test_relu_backward_bias_grad_views_and_errors(hip):
    """strided operands take the two-call road with the same results; shape errors and a bias gradient
    inside the gradient are refused"""
    from zenu_amd import _lib
    r = np.random.default_rng(3)
    M = hip.Matrix
    x = r.standard_normal((300, 96)).astype(np.float32)
    gy = r.standard_normal((300, 96)).astype(np.float32)
    X, GY = M.from_numpy(x), M.from_numpy(gy)
    xv, gv = X.slice(slice(0, 300, 2), slice(None)), GY.slice(slice(0, 300, 2), slice(None))   # every other row
    gx, gb = M.alloc((150, 96)), M.alloc((96,))
    gx.relu_backward_bias_grad(gb, gv, xv, 0.1)
    ref = gy[::2] * np.where(x[::2] > 0, np.float32(1), np.float32(0.1) * np.float32(-1))
    assert bits_equal(gx.to_numpy(), ref.astype(np.float32))
    assert np.allclose(gb.to_numpy(), ref.astype(np.float64).sum(0), rtol=1e-5, atol=1e-5)
    gb1 = M.alloc((1, 96))                                  # [1, N] is the same bias gradient
    gx.relu_backward_bias_grad(gb1, gv, xv, 0.1)
    assert bits_equal(gb1.to_numpy().reshape(-1), gb.to_numpy())
    with pytest.raises(_lib.ZenuHipError) as e:
        gx.relu_backward_bias_grad(M.alloc((95,)), gv, xv, 0.1)
    assert e.value.status == _lib.ERR_SHAPE
    with pytest.raises(_lib.ZenuHipError) as e:
        gx.relu_backward_bias_grad(gb, GY, xv, 0.1)
    assert e.value.status == _lib.ERR_SHAPE
    with pytest.raises(_lib.ZenuHipError) as e:
        gx.relu_backward_bias_grad(gx.index_axis(0, 0), gv, xv, 0.1)
    assert e.value.status == _lib.ERR_ARG


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("n,c", [(256, 10), (1, 4), (200, 16), (255, 13), (9, 1), (257, 10), (64, 17), (1000, 64)])
def test_cross_entropy_backward_bias_grad(hip, dtype, n, c):
    """gradient and its column sums from one call: the gradient is the bits of cross_entropy_backward,
    the column sums are within the bar of every sum of the oracle's sum_to and of the exact sums, and
    the same bits on every run; sizes on both sides of the one-launch conditions (<= 256 rows, <= 16 classes)"""
    print(f"[case] cross_entropy_backward_bias_grad {n}x{c} {np.dtype(dtype).name}", flush=True)
    r = np.random.default_rng(n * 17 + c)
    pred = r.standard_normal((n, c)).astype(dtype)
    ans = np.zeros((n, c), dtype=dtype)
    ans[np.arange(n), r.integers(0, c, n)] = 1
    M = hip.Matrix
    _, prob = hip.cross_entropy(M.from_numpy(pred), M.from_numpy(ans))
    p = prob.to_numpy()
    gl = np.array(1.75, dtype=dtype)
    for gloss in (None, gl):
        G = M.from_numpy(gloss) if gloss is not None else None
        gb = M.from_numpy(np.full(c, -3.0, dtype=dtype))
        g = hip.cross_entropy_backward_bias_grad(prob, M.from_numpy(ans), gb, G)
        g0 = hip.cross_entropy_backward(prob, M.from_numpy(ans), G)
        assert bits_equal(g.to_numpy(), g0.to_numpy())
        gbref = CpuMatrix.zeros((c,), dtype)
        gref = cpu_matrix.cross_entropy_backward_bias_grad(CpuMatrix.from_numpy(p), CpuMatrix.from_numpy(ans), gbref,
                                                           CpuMatrix.from_numpy(gloss) if gloss is not None else None)
        assert bits_equal(g.to_numpy(), gref.a)
        g64 = gref.a.astype(np.float64)
        exact = g64.sum(0)
        scale = np.maximum(np.abs(exact), np.abs(g64).sum(0) / np.sqrt(n))
        tol = 1e-5 if dtype == np.float32 else 1e-12
        assert np.all(np.abs(gb.to_numpy() - exact) <= tol * scale)
        assert np.all(np.abs(gb.to_numpy() - gbref.a) <= 2 * tol * scale)
        gb2 = M.alloc((c,), dtype)
        hip.cross_entropy_backward_bias_grad(prob, M.from_numpy(ans), gb2, G)
        assert bits_equal(gb2.to_numpy(), gb.to_numpy())


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_cross_entropy_head_every_small_geometry(hip, dtype):
    """every batch of 1..256 rows (at the wavefront and workgroup edges) with every class count 1..16 -- the
    geometries that the four-lanes-per-line kernels take: probabilities and gradients are the oracle's bits,
    the loss and the bias gradient within the bar of a sum"""
    M = hip.Matrix
    r = np.random.default_rng(77)
    tol = 1e-5 if dtype == np.float32 else 1e-12
    for n in (1, 2, 3, 4, 5, 63, 64, 65, 127, 128, 129, 191, 255, 256):
        for c in range(1, 17):
            pred = r.standard_normal((n, c)).astype(dtype) * 3
            ans = np.zeros((n, c), dtype=dtype)
            ans[np.arange(n), r.integers(0, c, n)] = 1
            loss_ref, prob_ref = cpu_matrix.cross_entropy(CpuMatrix.from_numpy(pred), CpuMatrix.from_numpy(ans))
            loss, prob = hip.cross_entropy(M.from_numpy(pred), M.from_numpy(ans))
            p = prob.to_numpy()
            assert bits_equal(p, prob_ref.a), (n, c)
            lr = float(loss_ref.a)
            assert abs(float(loss.to_numpy()) - lr) <= 4 * tol * max(abs(lr), 1e-30) + 1e-30, (n, c)
            gb = M.from_numpy(np.full(c, 9.0, dtype=dtype))
            g = hip.cross_entropy_backward_bias_grad(prob, M.from_numpy(ans), gb, None).to_numpy()
            gref = cpu_matrix.cross_entropy_backward(CpuMatrix.from_numpy(p), CpuMatrix.from_numpy(ans)).a
            assert bits_equal(g, gref), (n, c)
            g64 = gref.astype(np.float64)
            scale = np.maximum(np.abs(g64.sum(0)), np.abs(g64).sum(0) / np.sqrt(n))
            assert np.all(np.abs(gb.to_numpy() - g64.sum(0)) <= tol * scale + 1e-300), (n, c)


def test_cross_entropy_single_launch_equals_two_launches(hip):
    """up to 256 rows the cross-entropy forward folds its row terms in the workgroup that computed them;
    257 rows take the two-launch road: on the first 256 rows of the same data both give the same
    probabilities, and each loss is its own rows' exact value"""
    r = np.random.default_rng(8)
    pred = r.standard_normal((257, 10)).astype(np.float32)
    ans = np.zeros((257, 10), dtype=np.float32)
    ans[np.arange(257), r.integers(0, 10, 257)] = 1
    M = hip.Matrix
    la, pa = hip.cross_entropy(M.from_numpy(pred[:256]), M.from_numpy(ans[:256]))
    lb, pb = hip.cross_entropy(M.from_numpy(pred), M.from_numpy(ans))
    assert bits_equal(pa.to_numpy(), pb.to_numpy()[:256])
    for loss, rows in ((la, 256), (lb, 257)):
        lref, _ = cpu_matrix.cross_entropy(CpuMatrix.from_numpy(pred[:rows]), CpuMatrix.from_numpy(ans[:rows]))
        assert abs(float(loss.to_numpy()) - float(lref.a)) <= 4e-5 * abs(float(lref.a))
