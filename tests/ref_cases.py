"""Known-answer cases taken from the reference's own unit tests, written once and run on two
devices: the CPU oracle (tests/test_oracle_ref_cases.py, pins the oracle) and the HIP library
(tests/test_hip_ref_cases.py, GPU).  This mirrors run_mat_test! (zenu-test/src/lib.rs:62-91).

Each case names the reference test it restates.  `dev.M` is the matrix class (CpuMatrix or
zenu_amd.Matrix), `dev.sum_to` the sum_to function, `dev.Error` the "reference panics" exception.
Inputs and expected values are the reference's literals.
"""
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CASES = []


def case(fn):
    CASES.append(fn)
    return fn


def eq(m, expected, shape=None):
    got = m.to_numpy()
    exp = np.asarray(expected, dtype=got.dtype)
    if shape is not None:
        exp = exp.reshape(shape)
    assert got.shape == exp.shape, (got.shape, exp.shape)
    assert np.array_equal(got, exp), (got, exp)


def close(m, expected, eps, shape=None):
    got = m.to_numpy()
    exp = np.asarray(expected, dtype=np.float64)
    if shape is not None:
        exp = exp.reshape(shape)
    assert got.shape == exp.shape, (got.shape, exp.shape)
    assert np.max(np.abs(got.astype(np.float64) - exp)) <= eps, (got, exp)


R16 = [float(i) for i in range(1, 17)]
R8 = [1., 2., 3., 4., 5., 6., 7., 8.]

# ---- zenu-matrix/src/operation/basic_operations.rs:649-1335 -------------------------------------


@case
def scalar_add_1d(dev):  # basic_operations.rs:649
    a = dev.M.from_vec([1., 2., 3.], [3])
    ans = dev.M.zeros([3])
    ans.add_scalar(a, 1.)
    eq(ans, [2., 3., 4.])


@case
def scalar_add_2d(dev):  # :667
    a = dev.M.from_vec([1., 2., 3., 4., 5., 6.], [2, 3])
    ans = dev.M.zeros([2, 3])
    ans.add_scalar(a, 1.)
    eq(ans, [[2., 3., 4.], [5., 6., 7.]])


@case
def sliced_3d(dev):  # :689  slice_dynamic!(1.., .., ..;2)
    a = dev.M.from_vec(R16, [2, 2, 4])
    ans = dev.M.zeros([1, 2, 2])
    ans.add_scalar(a.slice(slice(1, None), slice(None), slice(None, None, 2)), 1.)
    eq(ans, [10., 12., 14., 16.], [1, 2, 2])


@case
def scalar_assign_4d(dev):  # :714
    a = dev.M.from_vec(R16, [2, 2, 2, 2])
    a.add_scalar_assign(1.)
    eq(a, [float(i) for i in range(2, 18)], [2, 2, 2, 2])


@case
def sliced_3d_assign(dev):  # :749  slice_dynamic!(2, 1..3, ..;2)
    v = [float(i * 100 + j * 10 + k) for i in range(3) for j in range(4) for k in range(5)]
    a = dev.M.from_vec(v, [3, 4, 5]).index_axis(0, 2).slice(slice(1, 3), slice(None, None, 2))
    ans = dev.M.zeros([2, 3])
    ans.add_scalar(a, 1.)
    eq(ans, [[211., 213., 215.], [221., 223., 225.]])


@case
def matrix_add_4d(dev):  # :780
    a = dev.M.from_vec(R16, [2, 2, 2, 2])
    b = dev.M.from_vec(R16[::-1], [2, 2, 2, 2])
    ans = dev.M.zeros([2, 2, 2, 2])
    ans.add_array(a, b)
    eq(ans, [17.] * 16, [2, 2, 2, 2])


@case
def matrix_add_sliced(dev):  # :823
    a = dev.M.from_vec(R16, [4, 4]).slice(slice(1, None, 2), slice(None, None, 2))
    b = dev.M.from_vec(R16, [4, 4]).slice(slice(None, None, 2), slice(1, None, 2))
    ans = dev.M.zeros([2, 2])
    ans.add_array(a, b)
    eq(ans, [[7., 11.], [23., 27.]])


@case
def transposed(dev):  # :856-889
    a = dev.M.from_vec(R16, [4, 4]).transpose()
    b = dev.M.from_vec(R16, [4, 4])
    ans = dev.M.zeros([4, 4])
    ans.add_array(a, b)
    eq(ans, [[2., 7., 12., 17.], [7., 12., 17., 22.], [12., 17., 22., 27.], [17., 22., 27., 32.]])


@case
def broadcast_add(dev):  # :900
    a = dev.M.from_vec(R8, [2, 2, 2])
    b = dev.M.from_vec([1., 1.], [1, 1, 2])
    ans = dev.M.zeros([2, 2, 2])
    ans.add_array(a, b)
    eq(ans, [2., 3., 4., 5., 6., 7., 8., 9.], [2, 2, 2])


@case
def add_2d_1d(dev):  # :925
    a = dev.M.from_vec(R8, [2, 2, 2])
    b = dev.M.from_vec([1., 1.], [2])
    ans = dev.M.zeros([2, 2, 2])
    ans.add_array(a, b)
    eq(ans, [2., 3., 4., 5., 6., 7., 8., 9.], [2, 2, 2])


@case
def add_2d_0d(dev):  # :950
    a = dev.M.from_vec(R8, [2, 2, 2])
    b = dev.M.from_vec([1.], [])
    ans = dev.M.zeros([2, 2, 2])
    ans.add_array(a, b)
    eq(ans, [2., 3., 4., 5., 6., 7., 8., 9.], [2, 2, 2])


@case
def broad_cast_4x1x1x1_4x3x3x3(dev):  # :975 (the lhs is the broadcast operand)
    a = dev.M.from_vec([1., 2., 3., 4.], [4, 1, 1, 1])
    b = dev.M.zeros([4, 2, 3, 3])
    ans = dev.M.zeros([4, 2, 3, 3])
    ans.add_array(a, b)
    exp = np.repeat(np.array([1., 2., 3., 4.], dtype=np.float32), 18).reshape(4, 2, 3, 3)
    eq(ans, exp)
    diff = ans - dev.M.from_numpy(exp)
    assert diff.asum() == 0.0


@case
def broadcast_add_1x4x1x1_3x4x5x5(dev):  # :1005
    a = dev.M.from_vec([1., 2., 3., 4.], [1, 4, 1, 1])
    b = dev.M.zeros([3, 4, 5, 5])
    ans = dev.M.zeros([3, 4, 5, 5])
    ans.add_array(a, b)
    exp = np.repeat(np.array([1., 2., 3., 4.], dtype=np.float32), 75).reshape(4, 3, 5, 5)
    result = dev.M.from_numpy(exp).transpose_by_index([1, 0, 2, 3])  # transpose_swap_index(0, 1)
    assert (ans - result).asum() == 0.0
    eq(ans, np.swapaxes(exp, 0, 1))


@case
def sub_mul_div_3d(dev):  # :1035-1335 (sub/mul/div x scalar/scalar_assign/array/assign)
    ones = [1.] * 8
    rev = R8[::-1]
    a = dev.M.from_vec(R8, [2, 2, 2]); ans = dev.M.zeros([2, 2, 2])
    ans.sub_scalar(a, 1.); eq(ans, [0., 1., 2., 3., 4., 5., 6., 7.], [2, 2, 2])
    a = dev.M.from_vec(R8, [2, 2, 2]); a.sub_scalar_assign(1.); eq(a, [0., 1., 2., 3., 4., 5., 6., 7.], [2, 2, 2])
    a = dev.M.from_vec(R8, [2, 2, 2]); ans.sub_array(a, dev.M.from_vec(ones, [2, 2, 2]))
    eq(ans, [0., 1., 2., 3., 4., 5., 6., 7.], [2, 2, 2])
    a.sub_assign(dev.M.from_vec(ones, [2, 2, 2])); eq(a, [0., 1., 2., 3., 4., 5., 6., 7.], [2, 2, 2])
    a = dev.M.from_vec(R8, [2, 2, 2]); ans.mul_scalar(a, 2.); eq(ans, [2., 4., 6., 8., 10., 12., 14., 16.], [2, 2, 2])
    a.mul_scalar_assign(2.); eq(a, [2., 4., 6., 8., 10., 12., 14., 16.], [2, 2, 2])
    a = dev.M.from_vec(R8, [2, 2, 2]); ans.mul_array(a, dev.M.from_vec(rev, [2, 2, 2]))
    eq(ans, [8., 14., 18., 20., 20., 18., 14., 8.], [2, 2, 2])
    a.mul_assign(dev.M.from_vec(rev, [2, 2, 2])); eq(a, [8., 14., 18., 20., 20., 18., 14., 8.], [2, 2, 2])
    a = dev.M.from_vec(R8, [2, 2, 2]); ans.div_scalar(a, 2.); eq(ans, [.5, 1., 1.5, 2., 2.5, 3., 3.5, 4.], [2, 2, 2])
    a.div_scalar_assign(2.); eq(a, [.5, 1., 1.5, 2., 2.5, 3., 3.5, 4.], [2, 2, 2])
    quot = np.array(R8, dtype=np.float32) / np.array(rev, dtype=np.float32)
    a = dev.M.from_vec(R8, [2, 2, 2]); ans.div_array(a, dev.M.from_vec(rev, [2, 2, 2])); eq(ans, quot, [2, 2, 2])
    a.div_assign(dev.M.from_vec(rev, [2, 2, 2])); eq(a, quot, [2, 2, 2])


@case
def sin_3d_and_sliced(dev):  # :1341, :1367
    a = dev.M.from_vec([0., 1., 2., 3., 4., 5., 6., 7.], [2, 2, 2])
    ans = dev.M.zeros([2, 2, 2])
    ans.sin_array(a)
    close(ans, np.sin(np.arange(8, dtype=np.float64)), 1e-6, [2, 2, 2])
    a = dev.M.from_vec([0., 1., 2., 3., 4., 5., 6., 7.], [8]).slice(slice(1, None, 2))
    ans = dev.M.zeros([4])
    ans.sin_array(a)
    close(ans, np.sin(np.array([1., 3., 5., 7.])), 1e-6)


@case
def pow_cases(dev):  # :1389 pow_1d, :1412 pow_0d, :1428 pow_2d_transposed
    a = dev.M.from_vec([0., 1., 2., 3., 4., 5., 6., 7.], [8])
    eq(a.powf_array(2.), [0., 1., 4., 9., 16., 25., 36., 49.])
    eq(dev.M.from_vec([4.], []).powf_array(2.), 16.)
    a = dev.M.from_vec(R8, [2, 4]).transpose()
    eq(a.powf_array(2.), [[1., 25.], [4., 36.], [9., 49.], [16., 64.]])


# ---- raw kernel tables: zenu-cuda/src/kernel/mod.rs:1015-1241 -------------------------------------

_UNARY_TABLE = [
    ("sin", [0.0, 1.0, 2.0, 3.0], [0.0, 0.8414709848078965, 0.9092974268256817, 0.1411200080598672]),
    ("cos", [0.0, 1.0, 2.0, 3.0], [1.0, 0.5403023058681398, -0.4161468365471424, -0.9899924966004454]),
    ("tan", [0.0, 1.0, 2.0, 3.0], [0.0, 1.5574077246549023, -2.185039863261519, -0.1425465430742778]),
    ("asin", [0.0, 0.5, 0.8, 1.0], [0.0, 0.5235987755982989, 0.9272952180016122, 1.5707963267948966]),
    ("acos", [0.0, 0.5, 0.8, 1.0], [1.5707963267948966, 1.0471975511965979, 0.6435011087932844, 0.0]),
    ("atan", [0.0, 0.5, 0.8, 1.0], [0.0, 0.4636476090008061, 0.6747409422235527, 0.7853981633974483]),
    ("sinh", [0.0, 0.5, 0.8, 1.0], [0.0, 0.5210953054937474, 0.888105982187623, 1.1752011936438014]),
    ("cosh", [0.0, 0.5, 0.8, 1.0], [1., 1.12762597, 1.33743495, 1.54308063]),
    ("tanh", [0.0, 0.5, 0.8, 1.0], [0.0, 0.46211715726000974, 0.6640367702678489, 0.7615941559557649]),
    ("abs", [-1.0, 0.5, -0.8, 1.0], [1.0, 0.5, 0.8, 1.0]),
    ("sqrt", [0.0, 0.5, 0.8, 1.0], [0.0, 0.7071067811865476, 0.8944271909999159, 1.0]),
    ("exp", [0.0, 0.5, 0.8, 1.0], [1.0, 1.6487212707001282, 2.225540928492468, 2.718281828459045]),
    ("log", [1.0, 2.0, 3.0], [0.0, 0.6931471805599453, 1.0986122886681098]),
]


@case
def unary_kernel_tables(dev):  # kernel/mod.rs:1015-1241, f32 and f64, out-of-place and in-place, 1e-6
    for name, xs, ys in _UNARY_TABLE:
        for dt in (np.float32, np.float64):
            a = dev.M.from_vec(xs, [len(xs)], dt)
            out = getattr(a, name)()
            close(out, ys, 1e-6)
            getattr(a, name + "_assign")()
            close(a, ys, 1e-6)


# ---- relu: relu.rs:255-296, zenu-cuda/src/kernel/activation.rs:88-147 -------------------------------


@case
def relu_cases(dev):
    x = dev.M.from_vec([1.0, -1.0, 0.0, 2.0], [2, 2])
    y = dev.M.zeros([2, 2])
    y.relu(x, 0.0)
    close(y, [[1.0, 0.0], [0.0, 2.0]], 1e-6)
    y.relu_backward_mask(x, 0.0)
    close(y, [[1.0, 0.0], [0.0, 1.0]], 1e-6)
    x0 = dev.M.from_vec([1.0], [])
    y0 = dev.M.zeros([])
    y0.relu(x0, 0.0)
    close(y0, 1.0, 1e-6)
    y0.relu_backward_mask(x0, 0.0)
    close(y0, 1.0, 1e-6)
    for dt in (np.float32, np.float64):  # activation.rs:88-147
        x = dev.M.from_vec([1.0, -1.0, 0.0, 2.0, -2.0], [5], dt)
        y = dev.M.zeros([5], dt)
        y.relu(x, 0.2)
        close(y, [1.0, -0.2, 0.0, 2.0, -0.4], 1e-6)
        y.relu_backward_mask(x, 0.1)
        close(y, [1.0, -0.1, -0.1, 1.0, -0.1], 1e-6)


# ---- sigmoid: zenu-autograd/src/activation/sigmoid.rs:26-66 --------------------------------------------


@case
def sigmoid_cases(dev):
    for dt in (np.float32, np.float64):
        x = dev.M.from_vec([0.0, 0.5, 0.1, 0.2, 0.3, 0.4], [2, 3], dt)
        close(x.sigmoid(), [[0.5, 0.62245935, 0.52497919], [0.54983399, 0.57444252, 0.59868766]], 1e-6)
        close(dev.M.from_vec([0.5], [], dt).sigmoid(), 0.62245935, 1e-6)


# ---- unary functions with their backward: zenu-autograd/src/functions/{tanh,sinh,cosh,powf,clip}.rs test mods ----

_X6 = [1., 2., 3., 4., 5., 6.]
_TANH6 = [0.7615941559557649, 0.9640275800758169, 0.9950547536867305, 0.999329299739067, 0.9999092042625951,
          0.9999877116507956]
_SINH6 = [1.1752011936438014, 3.626860407847019, 10.017874927409903, 27.28991719712775, 74.20321057778875,
          201.71315737027922]
_COSH6 = [1.5430806348152437, 3.7621956910836314, 10.067661995777765, 27.308232836016487, 74.20994852478785,
          201.7156361224559]


@case
def autograd_unary_backward(dev):
    # tanh_1d (tanh.rs test mod): y = tanh(x), x.grad = 1 / cosh(x)^2 with an all-ones output gradient, 1e-6
    x = dev.M.from_vec(_X6, [6])
    ones = dev.M.from_vec([1.] * 6, [6])
    close(x.tanh(), _TANH6, 1e-6)
    gx = dev.M.zeros([6])
    gx.tanh_backward(ones, x)
    close(gx, [1.0 / (c * c) for c in _COSH6], 1e-6)
    # sinh_1d / cosh_1d (f64): values, and gradients cosh(x) * gy / sinh(x) * gy (sinh.rs:30-35, cosh.rs)
    xd = dev.M.from_vec(_X6, [6], np.float64)
    od = dev.M.from_vec([1.] * 6, [6], np.float64)
    close(xd.sinh(), _SINH6, 1e-6 * 201.8)      # assert_val_eq's bound is on asum(diff) relative to the values' scale
    close(xd.cosh(), _COSH6, 1e-6 * 201.8)
    close(xd.cosh() * od, _COSH6, 1e-6 * 201.8)
    close(xd.sinh() * od, _SINH6, 1e-6 * 201.8)
    # powf_ (powf.rs test mod): x^2 and its gradient powf(x, factor - 1) * factor * gy (powf.rs:25-30)
    p = dev.M.from_vec([1., 2., 3.], [3])
    close(p.powf_array(2.0), [1., 4., 9.], 1e-6)
    two = dev.M.from_vec([2.0], [])
    close(p.powf_array(1.0) * two * dev.M.from_vec([1.] * 3, [3]), [2., 4., 6.], 1e-6)
    # clip_1d (clip.rs test mod)
    c = dev.M.from_vec(_X6, [6])
    eq(c.clip(2., 4.), [2., 2., 3., 4., 4., 4.])
    eq(c.clip_backward_mask(2., 4.), [0., 1., 1., 1., 0., 0.])
    # sigmoid backward has no test in the reference: closed form s (1 - s) at the sigmoid_cases points
    xs = dev.M.from_vec([0.0, 0.5, 0.1, 0.2, 0.3, 0.4], [6], np.float64)
    gs = dev.M.zeros([6], np.float64)
    gs.sigmoid_backward(dev.M.from_vec([1.] * 6, [6], np.float64), xs)
    sg = [0.5, 0.62245935, 0.52497919, 0.54983399, 0.57444252, 0.59868766]
    close(gs, [v * (1 - v) for v in sg], 1e-7)


# ---- stack / split: zenu-matrix/src/operation/stack.rs:71-108, split.rs:70-117 --------------------------------


@case
def stack_split_cases(dev):
    a, b, c = (dev.M.from_vec(v, [3]) for v in ([1., 2., 3.], [4., 5., 6.], [7., 8., 9.]))
    eq(dev.F.stack([a, b, c], 0), [1., 2., 3., 4., 5., 6., 7., 8., 9.])                        # test_stack_axis0
    a, b, c = (dev.M.from_vec(v, [2, 2]) for v in ([1., 2., 3., 4.], [5., 6., 7., 8.], [9., 10., 11., 12.]))
    eq(dev.F.stack([a, b, c], 1), [[1., 2., 5., 6., 9., 10.], [3., 4., 7., 8., 11., 12.]])     # test_stack_axis1
    parts = dev.F.split(dev.M.from_vec([1., 2., 3., 4., 5., 6.], [3, 2]), 0, 3)                # test_split_axis0
    assert len(parts) == 3
    for p, e in zip(parts, ([[1., 2.]], [[3., 4.]], [[5., 6.]])):
        eq(p, e)
    parts = dev.F.split(dev.M.from_vec([1., 2., 3., 4., 5., 6.], [2, 3]), 1, 3)                # test_split_axis1
    for p, e in zip(parts, ([[1.], [4.]], [[2.], [5.]], [[3.], [6.]])):
        eq(p, e)
    # a transposed input and a round trip: split(stack(x)) gives the inputs back
    t = dev.M.from_vec([1., 2., 3., 4., 5., 6.], [2, 3]).transpose()
    st = dev.F.stack([t, t], 0)
    eq(st, [[1., 4.], [2., 5.], [3., 6.], [1., 4.], [2., 5.], [3., 6.]])
    for p in dev.F.split(st, 0, 2):
        eq(p, [[1., 4.], [2., 5.], [3., 6.]])


# ---- mean / variance: zenu-matrix/src/operation/var.rs test mod, mean.rs:9-20 ------------------------------


@case
def mean_variance_cases(dev):
    for dt in (np.float32, np.float64):
        close(dev.M.from_vec([1., 2., 3., 4.], [4], dt).variance(None, False), 1.25, 1e-6)      # variance_1d
        close(dev.M.from_vec([1., 2.], [2], dt).variance(None, False), 0.25, 1e-6)              # variance_1d_
        x = dev.M.from_vec([1., 2., 3., 4.], [2, 2], dt)
        close(x.variance(None, False), 1.25, 1e-6)                                              # variance_2d
        close(x.variance(0, False), [1., 1.], 1e-6)                                             # variance_2d_0
        close(x.variance(1, False), [0.25, 0.25], 1e-6)                                         # variance_2d_1
        close(x.mean(0, False), [2., 3.], 1e-6)
        close(x.mean(1, True), [[1.5], [3.5]], 1e-6)
        # without an axis the reference averages |x| (mean.rs:15-19 calls asum)
        close(dev.M.from_vec([-1., 2., -3., 4.], [4], dt).mean(None, False), 2.5, 1e-6)


# ---- sum: sum.rs:109-245 ------------------------------------------------------------------------------

_SUM1 = [60, 63, 66, 69, 72, 75, 78, 81, 84, 87, 90, 93, 96, 99, 102, 105, 108, 111, 114, 117,
         240, 243, 246, 249, 252, 255, 258, 261, 264, 267, 270, 273, 276, 279, 282, 285, 288, 291, 294, 297]
_SUM2 = [30, 34, 38, 42, 46, 110, 114, 118, 122, 126, 190, 194, 198, 202, 206, 270, 274, 278,
         282, 286, 350, 354, 358, 362, 366, 430, 434, 438, 442, 446]
_SUM3 = [10, 35, 60, 85, 110, 135, 160, 185, 210, 235, 260, 285, 310, 335, 360, 385, 410, 435,
         460, 485, 510, 535, 560, 585]


@case
def sum_4d(dev):  # test_4d :109, test_4d_keep_dim :176
    for dt in (np.float32, np.float64):
        src = dev.M.from_vec([float(i) for i in range(120)], [2, 3, 4, 5], dt)
        ans0 = [float(i) for i in range(60, 179) if i % 2 == 0]
        for keep in (False, True):
            def shp(axis):
                s = [2, 3, 4, 5]
                if keep:
                    s[axis] = 1
                else:
                    del s[axis]
                return s
            eq(src.sum(0, keep), ans0, shp(0))
            eq(src.sum(1, keep), _SUM1, shp(1))
            eq(src.sum(2, keep), _SUM2, shp(2))
            eq(src.sum(3, keep), _SUM3, shp(3))


@case
def sum_to_cases(dev):  # zenu-autograd/src/functions/sum_to.rs:63-74 and sum.rs:35-94 branches
    src = dev.M.from_vec([1., 2., 3., 4., 5., 6.], [2, 3])
    t = dev.M.zeros([3]); dev.sum_to(src, t); eq(t, [5., 7., 9.])
    t = dev.M.zeros([]); dev.sum_to(src, t); eq(t, 21.)
    t = dev.M.zeros([2, 1]); dev.sum_to(src, t); eq(t, [[6.], [15.]])
    t = dev.M.zeros([1, 3]); dev.sum_to(src, t); eq(t, [[5., 7., 9.]])
    t = dev.M.zeros([1, 1]); dev.sum_to(src, t); eq(t, [[21.]])
    t = dev.M.zeros([2, 3]); dev.sum_to(src, t); eq(t, [[1., 2., 3.], [4., 5., 6.]])
    src4 = dev.M.from_vec([float(i) for i in range(120)], [2, 3, 4, 5])
    t = dev.M.zeros([4, 5]); dev.sum_to(src4, t)
    eq(t, np.arange(120, dtype=np.float32).reshape(2, 3, 4, 5).sum(axis=(0, 1)))


# ---- max: max.rs:157-844 --------------------------------------------------------------------------------


@case
def max_idx_cases(dev):  # default_1d :157, default_2d :168, sliced_3d :179
    assert tuple(dev.M.from_vec([0., 1., 2., 3.], [4]).max_idx()) == (3,)
    assert tuple(dev.M.from_vec([0., 1., 2., 3.], [2, 2]).max_idx()) == (1, 1)
    a = dev.M.from_vec([float(i) for i in range(512)], [8, 8, 8])
    sliced = a.slice(slice(None, None, 3), slice(None, None, 4), slice(None, None, 2))
    assert tuple(sliced.max_idx()) == (2, 1, 3)
    assert sliced.max_item() == 6 * 64 + 4 * 8 + 6


_MAX_REVAL = [0.04881350392732475, 0.21518936637241948, 0.10276337607164387, 0.044883182996896864,
              -0.07634520066109529, 0.14589411306665612, -0.06241278873730749, 0.39177300078207977,
              0.4636627605010293, -0.1165584811742223, 0.2917250380826646, 0.02889491975290448,
              0.06804456109393231, 0.42559663829266103, -0.42896394180211306, -0.4128707002984593,
              -0.4797816025596743, 0.332619845547938, 0.2781567509498505, 0.37001214824681916,
              0.478618342232764, 0.2991585642167236, -0.038520637747068154, 0.28052917628645546]


@case
def max_axis_reval(dev):  # :204-245
    m = dev.M.from_vec(_MAX_REVAL, [2, 3, 4])
    assert m.max_axis_idx_ravel(0) == [1, 1, 0, 0, 0, 1, 1, 0, 1, 1, 0, 1]
    assert m.max_axis_idx_ravel(1) == [2, 0, 2, 1, 2, 0, 1, 1]
    assert m.max_axis_idx_ravel(2) == [1, 3, 0, 1, 3, 0]


@case
def max_axis_4d(dev):  # :247-545 (f32) and :546-844 (f64); vectors in tests/golden/*.json
    for name, dt in (("max_axis_4d_f32.json", np.float32), ("max_axis_4d_f64.json", np.float64)):
        g = json.load(open(os.path.join(GOLDEN, name)))
        m = dev.M.from_vec(g["input"], g["shape"], dt)
        close(m.max_axis(0, False), g["ans_0d"], 1e-6, [3, 4, 5])
        close(m.max_axis(1, False), g["ans_1d"], 1e-6, [2, 4, 5])
        close(m.max_axis(2, False), g["ans_2d"], 1e-6, [2, 3, 5])
        close(m.max_axis(3, False), g["ans_3d"], 1e-6, [2, 3, 4])
        assert m.max_axis(1, True).shape == (2, 1, 4, 5)


# ---- asum: asum.rs:78-120 ---------------------------------------------------------------------------------


@case
def asum_cases(dev):  # defualt_1d :78, defualt_2d :90, sliced_2d :102
    assert dev.M.from_vec([1.0, 2.0, 3.0], [3]).asum() == 6.0
    a = dev.M.from_vec([1.0, 2.0, 3.0, 4.0], [2, 2])
    assert a.asum() == 10.0
    assert a.slice(slice(0, 2), slice(0, 1)).asum() == 4.0
    # not in the reference's tests, fixed by its code: |x| is summed on contiguous views ...
    assert dev.M.from_vec([1.0, -2.0, 3.0, -4.0], [2, 2]).asum() == 10.0
    # ... but a 0-d view returns the raw item (asum.rs:52-53) and a view none of whose trailing
    # sub-views is contiguous recurses down to 0-d items, i.e. a plain sum (asum.rs:59-65)
    assert dev.M.from_vec([-3.0], []).asum() == -3.0
    assert dev.M.from_vec([1.0, 9.0, -2.0, 9.0], [4]).slice(slice(None, None, 2)).asum() == -1.0


# ---- with_clousers.rs:356-508 (results; the call counts are checked on the oracle only) ------------------


@case
def with_closures_results(dev):
    a = dev.M.zeros([10, 10, 10]); a.add_scalar_assign(1.0); eq(a, np.ones((10, 10, 10)))
    a = dev.M.zeros([2, 4, 5])
    a.slice(slice(None), slice(None, None, 2), slice(None)).add_scalar_assign(1.0)
    exp = np.zeros((2, 4, 5), dtype=np.float32); exp[:, ::2, :] = 1.0
    eq(a, exp)
    a = dev.M.zeros([10, 10, 10]); a.add_assign(dev.M.from_vec([1.0] * 1000, [10, 10, 10])); eq(a, np.ones((10, 10, 10)))
    a = dev.M.zeros([10, 10, 10]); a.add_assign(dev.M.from_vec([1.0] * 100, [10, 10])); eq(a, np.ones((10, 10, 10)))
    b_np = np.arange(1000, dtype=np.float32).reshape(10, 10, 10)
    a = dev.M.zeros([10, 10, 10]); a.add_assign(dev.M.from_numpy(b_np).index_axis(1, 2))
    eq(a, np.broadcast_to(b_np[:, 2, :], (10, 10, 10)))
    a = dev.M.zeros([20, 10, 10]); bv = np.arange(100, dtype=np.float32).reshape(10, 10)
    a.slice(slice(None, None, 2), slice(None), slice(None)).add_assign(dev.M.from_numpy(bv))
    exp = np.zeros((20, 10, 10), dtype=np.float32); exp[::2] = bv
    eq(a, exp)
    a = dev.M.zeros([2, 4, 5]); b = dev.M.from_vec([1.0] * 40, [2, 4, 5])
    sl = (slice(None), slice(None, None, 2), slice(None))
    a.slice(*sl).add_scalar(b.slice(*sl), 2.0)
    exp = np.zeros((2, 4, 5), dtype=np.float32); exp[:, ::2, :] = 3.0
    eq(a, exp)
    a = dev.M.zeros([10, 10, 10])
    a.add_array(dev.M.from_vec([1.0] * 1000, [10, 10, 10]), dev.M.from_vec([2.0] * 1000, [10, 10, 10]))
    eq(a, np.full((10, 10, 10), 3.0))


# ---- copy_from / to_default_stride: copy_from.rs:285-398, to_default_stride.rs:28-89 -----------------------


@case
def copy_cases(dev):
    v = np.arange(16, dtype=np.float32)
    a = dev.M.from_numpy(v).slice(slice(None, None, 2))        # 1-D stride 2
    eq(a.to_default_stride(), v[::2])
    m = dev.M.from_numpy(v.reshape(4, 4))
    eq(m.slice(slice(None, None, 2), slice(1, None, 2)).to_default_stride(), v.reshape(4, 4)[::2, 1::2])
    eq(m.transpose().to_default_stride(), v.reshape(4, 4).T)
    t3 = np.arange(18, dtype=np.float32).reshape(2, 3, 3) + 1
    eq(dev.M.from_numpy(t3).transpose_by_index([2, 1, 0]).to_default_stride().reshape([18]),
       [1., 10., 4., 13., 7., 16., 2., 11., 5., 14., 8., 17., 3., 12., 6., 15., 9., 18.])  # reshape.rs:154-172
    dst = dev.M.zeros([4, 4])
    dst.slice(slice(None, None, 2), slice(None)).copy_from(m.slice(slice(2, None), slice(None)))
    exp = np.zeros((4, 4), dtype=np.float32); exp[::2] = v.reshape(4, 4)[2:]
    eq(dst, exp)


# ---- legality: with_clousers.rs:42-50,87-107,155-178, dim_dyn.rs:24-58 ---------------------------------------


@case
def shape_errors(dev):
    import pytest
    with pytest.raises(dev.Error):   # [4,1] + [1,4]: no mutual broadcasting
        dev.M.zeros([4, 4]).add_array(dev.M.zeros([4, 1]), dev.M.zeros([1, 4]))
    with pytest.raises(dev.Error):   # lower rank must match trailing dims exactly
        dev.M.zeros([2, 3, 4]).add_array(dev.M.zeros([2, 3, 4]), dev.M.zeros([1, 4]))
    with pytest.raises(dev.Error):   # destination must have the larger shape
        dev.M.zeros([3]).add_array(dev.M.zeros([2, 3]), dev.M.zeros([3]))
    with pytest.raises(dev.Error):   # rank(to) < rank(rhs)
        dev.M.zeros([3]).add_assign(dev.M.zeros([2, 3]))
    with pytest.raises(dev.Error):   # not include-broadcast
        dev.M.zeros([2, 3]).add_assign(dev.M.zeros([2, 2]))
    with pytest.raises(dev.Error):   # unary shape mismatch
        dev.M.zeros([2, 3]).exp_array(dev.M.zeros([3, 2]))
    with pytest.raises(dev.Error):   # Invalid axis
        dev.M.zeros([2, 3]).sum(2)
    with pytest.raises(dev.Error):
        dev.M.zeros([2, 3]).max_axis(5)


# ---- softmax / cross-entropy / clip: the chains the fused entry points replace --------------------
# `dev.F` holds softmax_backward, cross_entropy, cross_entropy_backward (op-by-op on the CPU device)


@case
def softmax_cases(dev):  # zenu-matrix/src/operation/softmax.rs:37-91 (softmax_1d, softmax_2d), 1e-6 on asum
    a = dev.M.from_vec([1., 2., 3., 4.], [4])
    b = dev.M.zeros([4])
    b.softmax_assign(a, 0)
    ans = dev.M.from_vec([0.0320586, 0.08714432, 0.23688284, 0.64391428], [4])
    assert (b - ans).asum() < 1e-6
    a = dev.M.from_vec([1., 2., 3., 4., 5., 6.], [2, 3])
    b = dev.M.zeros([2, 3])
    b.softmax_assign(a, 1)
    ans = dev.M.from_vec([0.09003057, 0.24472847, 0.66524096, 0.09003057, 0.24472847, 0.66524096], [2, 3])
    assert (b - ans).asum() < 1e-6
    b = dev.M.zeros([2, 3])
    b.softmax_assign(a, 0)
    ans = dev.M.from_vec([0.04742587, 0.04742587, 0.04742587, 0.95257413, 0.95257413, 0.95257413], [2, 3])
    assert (b - ans).asum() < 1e-6
    with_axis_error = False
    try:
        b.softmax_assign(a, 2)      # "axis must be less than the number of dimensions"
    except dev.Error:
        with_axis_error = True
    assert with_axis_error


@case
def softmax_backward_2d_1d(dev):  # zenu-autograd/src/loss/softmax.rs:70-103, f64, 1e-6
    x = dev.M.from_vec([1., 2., 3., 4., 5., 6., 7., 8.], [2, 4], np.float64)
    y = dev.M.zeros([2, 4], np.float64)
    y.softmax_assign(x, 1)
    close(y, [0.0320586, 0.08714432, 0.23688284, 0.64391428] * 2, 1e-6, (2, 4))
    # loss = sum(y * [1,2,3,4]) => the gradient arriving at y is [1,2,3,4] in every row
    gy = dev.M.from_vec([1., 2., 3., 4.] * 2, [2, 4], np.float64)
    gx = dev.F.softmax_backward(y, gy, 1)
    close(gx, [-0.07991097, -0.13007621, -0.11670097, 0.32668814] * 2, 1e-6, (2, 4))


@case
def cross_entropy_cases(dev):  # zenu-autograd/src/loss/cross_entropy.rs:38-84
    pred = dev.M.from_vec([0.1, 0.9, 0.1, 0.1], [1, 4], np.float64)
    ans = dev.M.from_vec([0., 1., 0., 0.], [1, 4], np.float64)
    loss, prob = dev.F.cross_entropy(pred, ans)
    close(loss, 0.8536, 1e-4)
    close(dev.F.cross_entropy_backward(prob, ans), [[0.1914, -0.5741, 0.1914, 0.1914]], 1e-4)
    pred = dev.M.from_vec([0.1, 0.9, 0.1, 0.1, 0.01, 0.9, 0.2, 0.05], [2, 4])
    ans = dev.M.from_vec([0., 1., 0., 0., 1., 0., 0., 0.], [2, 4])
    loss, prob = dev.F.cross_entropy(pred, ans)
    close(loss, 1.2957, 2e-5)
    close(dev.F.cross_entropy_backward(prob, ans),
          [[0.0957, -0.2871, 0.0957, 0.0957], [-0.4121, 0.2142, 0.1064, 0.0915]], 3e-4)


@case
def clip_cases(dev):  # zenu-matrix/src/operation/clip.rs:321-372; zenu-cuda/src/kernel/mod.rs:1300-1368
    for shape in ([4], [2, 2]):
        a = dev.M.from_vec([1., 2., 3., 4.], shape)
        eq(a.clip(2., 3.), [2., 2., 3., 3.], shape)
        a.clip_assign(2., 3.)
        eq(a, [2., 2., 3., 3.], shape)
    for dt in (np.float32, np.float64):
        a = dev.M.from_vec([0., 1., 2., 3., 4., 5.], [6], dt)
        eq(a.clip_backward_mask(1., 2.), [0., 1., 1., 0., 0., 0.])
        a.clip_backward_assign_mask(1., 2.)
        eq(a, [0., 1., 1., 0., 0., 0.])


@case
def view_cases(dev):  # zenu-matrix/src/operation/transpose.rs:70-206, reshape.rs:108-176, add_axis.rs:25-33
    M = dev.M
    # transpose_2d: [[1,2,3],[4,5,6]] transposed, read element by element
    a = M.from_numpy(np.array([1., 2., 3., 4., 5., 6.], dtype=np.float32).reshape(2, 3)).transpose()
    got = a.to_default_stride().to_numpy()
    assert got.shape == (3, 2)
    for (i, j), v in {(0, 0): 1., (0, 1): 4., (1, 0): 2., (1, 1): 5., (2, 0): 3., (2, 1): 6.}.items():
        assert got[i, j] == v
    # inplace_transpose_4d: element (i, j, k, l) = 1000 i + 100 j + 10 k + l on [3,4,5,6]; transpose_by_index
    # [1,0,2,3] into a new matrix.  The reference's literal lists the result row by row: [4,3,5,6] with
    # element (j, i, k, l) = 1000 i + 100 j + 10 k + l (its first rows: 0..5, 10..15, ..., 40..45, 1000..1005).
    i, j, k, l = np.meshgrid(np.arange(3), np.arange(4), np.arange(5), np.arange(6), indexing="ij")
    x = (1000 * i + 100 * j + 10 * k + l).astype(np.float32)
    out = M.from_numpy(x).transpose_by_index([1, 0, 2, 3]).to_default_stride()
    ans = np.empty((4, 3, 5, 6), dtype=np.float32)
    for jj in range(4):
        for ii in range(3):
            for kk in range(5):
                for ll in range(6):
                    ans[jj, ii, kk, ll] = 1000 * ii + 100 * jj + 10 * kk + ll
    assert list(ans.reshape(-1)[:12]) == [0., 1., 2., 3., 4., 5., 10., 11., 12., 13., 14., 15.]     # the literal's first entries
    assert list(ans.reshape(-1)[30:36]) == [1000., 1001., 1002., 1003., 1004., 1005.]
    eq(out, ans)
    # swap_axis (2-d) and swap_axis_3d: transpose_swap_index_new_matrix(0, 1)
    eq(M.from_numpy(np.array([1., 2., 3., 4., 5., 6.], dtype=np.float32).reshape(2, 3)).transpose_by_index([1, 0]).to_default_stride(),
       [1., 4., 2., 5., 3., 6.], (3, 2))
    x3 = np.arange(1, 25, dtype=np.float32).reshape(2, 3, 4)
    eq(M.from_numpy(x3).transpose_by_index([1, 0, 2]).to_default_stride(),
       [1., 2., 3., 4., 13., 14., 15., 16., 5., 6., 7., 8., 17., 18., 19., 20., 9., 10., 11., 12., 21., 22., 23., 24.], (3, 2, 4))
    # reshape_3d_1d, reshape_1d_3d: views of the same data
    r18 = np.arange(1, 19, dtype=np.float32)
    eq(M.from_numpy(r18.reshape(2, 3, 3)).reshape([18]), r18, (18,))
    eq(M.from_numpy(np.arange(1, 7, dtype=np.float32)).reshape([2, 3, 1]), [1., 2., 3., 4., 5., 6.], (2, 3, 1))
    # reshape_new_matrix_3d_1d: transpose_by_index [2,1,0], then a new default-stride matrix reshaped to [18]
    eq(M.from_numpy(r18.reshape(2, 3, 3)).transpose_by_index([2, 1, 0]).to_default_stride().reshape([18]),
       [1., 10., 4., 13., 7., 16., 2., 11., 5., 14., 8., 17., 3., 12., 6., 15., 9., 18.], (18,))
    # add_axis: [2,2] -> [1,2,2], same data; a - ans has asum 0
    a = M.from_numpy(np.array([1., 2., 3., 4.], dtype=np.float32).reshape(2, 2)).add_axis(0)
    assert tuple(a.shape) == (1, 2, 2)
    ans = M.from_numpy(np.array([1., 2., 3., 4.], dtype=np.float32).reshape(1, 2, 2))
    assert float((a - ans).asum()) == 0.0


@case
def broadcast_cases(dev):  # zenu-matrix/src/operation/broadcast.rs:53-165
    for src, sshape, dshape in (([1.], [], [3]), ([1.], [], [2, 3]), ([1., 2., 3.], [3], [2, 3]),
                                ([1., 2.], [1, 2], [2, 3, 1, 2]), ([1., 2., 3., 4.], [1, 1, 1, 4], [2, 3, 4, 4])):
        s = dev.M.from_vec(src, sshape)
        res = dev.M.zeros(dshape)
        res.broadcast(s)
        eq(res, np.broadcast_to(np.asarray(src, dtype=np.float32).reshape(sshape), dshape))
    # the first is refused by the test at broadcast.rs:13-17; the others pass it and fail in the
    # recursion (a copy_from between different shapes, or the same test one level down)
    for dshape, sshape in (([2, 3], [2]), ([2, 3], [2, 1]), ([2, 4, 3, 3], [1, 4, 1, 1]), ([2, 2, 3], [2, 1, 3])):
        n = int(np.prod(sshape))
        bad = False
        try:
            dev.M.zeros(dshape).broadcast(dev.M.from_vec([1.] * n, sshape))
        except dev.Error:
            bad = True
        assert bad, (dshape, sshape)
