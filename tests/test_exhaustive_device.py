"""Every f32 bit pattern through the elementwise kernels, results copied back and compared element by
element: the twelve functions whose results are meant to be the host libm's bits, the one that is
allowed a distance (tanh_ulp2: 2 ulp), powf for seven exponents, f64 sweeps and tensors
beyond 2^31 / 2^32 elements.

Opt-in (ZENU_EXHAUSTIVE=1): moving 2^32 results to the host and comparing them there takes half a minute
per function.  The default suite compares the twelve bit-exact functions on all 2^32 arguments too, but
through sums folded on the device and on the host (test_hip_parity.py::
test_every_f32_argument_equals_the_host_libm, two seconds per function), and every 16th pattern element by
element; the host build of the same source is compared on every 31st pattern (test_host_native.py).  Run as
    ZENU_EXHAUSTIVE=1 python -u -m pytest tests/test_exhaustive_device.py -m gpu -x -s --timeout 3000
"""
import os
from concurrent.futures import ThreadPoolExecutor

import numpy as np
import pytest

import zenu_oracle as zo

pytestmark = [pytest.mark.gpu,
              pytest.mark.skipif(os.environ.get("ZENU_EXHAUSTIVE") != "1", reason="opt-in: set ZENU_EXHAUSTIVE=1")]

CHUNK = 1 << 26
THREADS = 16

# (Matrix method, oracle function id or None for the sigmoid composite, largest allowed distance in ulp)
FUNCTIONS = [("tanh", zo.TANH, 0), ("sigmoid", None, 0), ("exp", zo.EXP, 0), ("log", zo.LOG, 0),
             ("sinh", zo.SINH, 0), ("cosh", zo.COSH, 0), ("sin", zo.SIN, 0), ("cos", zo.COS, 0),
             ("asin", zo.ASIN, 0), ("acos", zo.ACOS, 0), ("atan", zo.ATAN, 0), ("tanh_ulp2", zo.TANH, 2),
             ("tan", zo.TAN, 0)]


def oracle_chunk(fn, x, exponent=None):
    """the oracle (the host libm behind the reference's CPU path) on a chunk, split over threads;
    ctypes releases the interpreter lock during each call"""
    out = np.empty_like(x)
    step = x.size // THREADS

    def part(i):
        sl = slice(i * step, x.size if i == THREADS - 1 else (i + 1) * step)
        if exponent is not None:
            zo.powf(out[sl], x[sl], exponent)
        elif fn is None:
            zo.sigmoid(out[sl], x[sl])
        else:
            zo.unary(fn, out[sl], x[sl])
    with ThreadPoolExecutor(THREADS) as pool:
        list(pool.map(part, range(THREADS)))
    return out


def ordered(a):
    i = a.view(np.int32).astype(np.int64)
    return np.where(i < 0, np.int64(-2**31) - i, i)


@pytest.mark.parametrize("name,fn,bar", FUNCTIONS)
def test_all_f32_bit_patterns(hip, name, fn, bar):
    worst, differing, total = 0, 0, 0
    with np.errstate(all="ignore"):
        for start in range(0, 1 << 32, CHUNK):
            x = np.arange(start, start + CHUNK, dtype=np.uint64).astype(np.uint32).view(np.float32)
            got = getattr(hip.Matrix.from_numpy(x), name)().to_numpy()
            exp = oracle_chunk(fn, x)
            nan = np.isnan(exp)
            assert np.array_equal(np.isnan(got), nan), f"{name}: NaN positions differ in chunk {start:#x}"
            ok = ~nan
            if bar == 0:
                bad = got.view(np.uint32)[ok] != exp.view(np.uint32)[ok]
                if bad.any():
                    i = np.flatnonzero(ok)[np.flatnonzero(bad)[0]]
                    raise AssertionError(f"{name}: {int(bad.sum())} of {CHUNK} differ in chunk {start:#x}, first x = "
                                         f"{x[i]!r} ({x.view(np.uint32)[i]:#010x}): got {got[i]!r}, libm {exp[i]!r}")
            else:
                d = np.abs(ordered(got[ok]) - ordered(exp[ok]))
                worst = max(worst, int(d.max()))
                differing += int((d > 0).sum())
                assert worst <= bar, f"{name}: {worst} ulp in chunk {start:#x}"
            total += int(ok.sum())
            if start % (1 << 30) == 0:
                print(f"[exhaustive] {name}: {start >> 26} of 64 chunks", flush=True)
    print(f"[exhaustive] {name}: {total} arguments, largest distance {worst} ulp, {differing} differ", flush=True)


@pytest.mark.parametrize("exponent", [2.0, 0.5, 2.5, -1.0, 3.0, -0.5, 1.0 / 3.0])
def test_powf_all_bases(hip, exponent):
    """powf(x, exponent) for every f32 base (negative bases, zeros, subnormals, infinities and NaN included)"""
    total = 0
    with np.errstate(all="ignore"):
        for start in range(0, 1 << 32, CHUNK):
            x = np.arange(start, start + CHUNK, dtype=np.uint64).astype(np.uint32).view(np.float32)
            got = hip.Matrix.from_numpy(x).powf_array(exponent).to_numpy()
            exp = oracle_chunk(None, x, exponent)
            nan = np.isnan(exp)
            assert np.array_equal(np.isnan(got), nan), f"powf {exponent}: NaN positions differ in chunk {start:#x}"
            ok = ~nan
            bad = got.view(np.uint32)[ok] != exp.view(np.uint32)[ok]
            if bad.any():
                i = np.flatnonzero(ok)[np.flatnonzero(bad)[0]]
                raise AssertionError(f"powf {exponent}: {int(bad.sum())} differ in chunk {start:#x}, first x = {x[i]!r}: "
                                     f"got {got[i]!r}, libm {exp[i]!r}")
            total += int(ok.sum())
            if start % (1 << 30) == 0:
                print(f"[exhaustive] powf {exponent}: {start >> 26} of 64 chunks", flush=True)
    print(f"[exhaustive] powf(x, {exponent}): {total} bases, 0 differ", flush=True)


@pytest.mark.parametrize("name,fn", [("tanh", zo.TANH), ("sigmoid", None), ("exp", zo.EXP), ("sinh", zo.SINH),
                                     ("cosh", zo.COSH), ("log", zo.LOG), ("sin", zo.SIN), ("cos", zo.COS),
                                     ("powf 2.5", 2.5), ("powf -3.0", -3.0), ("powf 0.3", 0.3)])
def test_f64_every_fourth_high_word(hip, name, fn):
    """f64 cannot be exhausted: every 4th value of the high word (sign, exponent, 20 mantissa bits) with a
    pseudo-random low word, 2^30 arguments per function (ZENU_EXHAUSTIVE_F64_LOG2=33: eight times as many,
    with other low words), must give the host libm's bits"""
    total = 0
    n = 1 << 25
    passes = 1 << max(0, int(os.environ.get("ZENU_EXHAUSTIVE_F64_LOG2", "30")) - 30)   # more low words on request
    with np.errstate(all="ignore"):
        for c in range(32 * passes):
            rep, c = divmod(c, 32)
            hi = (np.arange(c * n, (c + 1) * n, dtype=np.uint64) * 4 + ((c + rep) & 3)) & 0xffffffff
            lo = ((hi + np.uint64(rep)) * np.uint64(0x9E3779B97F4A7C15 + 2 * rep) >> np.uint64(29)) & np.uint64(0xffffffff)
            x = ((hi << np.uint64(32)) | lo).view(np.float64)
            if name.startswith("powf"):
                got = hip.Matrix.from_numpy(x).powf_array(fn).to_numpy()
                exp = oracle_chunk(None, x, exponent=fn)
            else:
                got = getattr(hip.Matrix.from_numpy(x), name)().to_numpy()
                exp = oracle_chunk(fn, x)
            nan = np.isnan(exp)
            assert np.array_equal(np.isnan(got), nan), f"{name} f64: NaN positions differ in chunk {c}"
            ok = ~nan
            bad = got.view(np.uint64)[ok] != exp.view(np.uint64)[ok]
            if bad.any():
                i = np.flatnonzero(ok)[np.flatnonzero(bad)[0]]
                raise AssertionError(f"{name} f64: {int(bad.sum())} differ in chunk {c}, first x = {x[i]!r} "
                                     f"({x.view(np.uint64)[i]:#018x}): got {got[i]!r}, libm {exp[i]!r}")
            total += int(ok.sum())
            if c % 8 == 0:
                print(f"[exhaustive] {name} f64: pass {rep}, {c} of 32 chunks", flush=True)
    print(f"[exhaustive] {name} f64: {total} arguments, 0 differ", flush=True)


def test_beyond_2_31_and_2_32_elements(hip):
    """index arithmetic past 32 bits: tensors of 2^31 + 4099 and of 65537 x 65540 (> 2^32) f32 elements, built
    and checked on the device (only small slices come back): fills, scalar and row-broadcast operators,
    out-of-place multiply, first-maximum search, sums along both axes and over everything"""
    M = hip.Matrix
    n = (1 << 31) + 4099
    A = M.zeros((n,))
    A.add_scalar_assign(1.0)
    A.slice(slice(n - 1, n)).copy_from(M.from_numpy(np.array([5.0], dtype=np.float32)))
    A.slice(slice(n - 3000, n - 2999)).copy_from(M.from_numpy(np.array([5.0], dtype=np.float32)))
    with pytest.raises(hip.ZenuHipError):                 # positions are tracked in 32 bits: a reduced length of
        A.max_idx()                                       # 2^31 - 1 or more is refused, never answered wrongly
    V = M(A.buf, A.offset + 4099, (2, 1 << 30), (1 << 30, 1), A.dtype)   # the last 2^31 elements as two rows
    assert V.max_axis_idx_ravel(1) == [0, (1 << 30) - 3000]   # the first of the two maxima of the second row
    B = A * 2.0
    head, tail = B.slice(slice(0, 8)).to_numpy(), B.slice(slice(n - 8, n)).to_numpy()
    assert np.array_equal(head, np.full(8, 2.0, np.float32))
    assert np.array_equal(tail, np.array([2.0] * 7 + [10.0], dtype=np.float32))
    total = float(A.sum(0).to_numpy())
    assert abs(total - (n + 8.0)) <= 1e-5 * n
    print("[exhaustive] 2^31 + 4099 elements: ok", flush=True)
    del A, B

    rows, cols = 65537, 65540                             # 4 295 295 980 elements, 16 GiB
    X = M.zeros((rows, cols))
    X.add_scalar_assign(1.0)
    row = M.from_numpy(np.arange(cols, dtype=np.float32).reshape(1, cols) % 7)
    X.add_assign(row)                                     # too long for the 32-bit flat kernel: the row kernel
    exp_row = (np.arange(cols) % 7 + 1).astype(np.float32)
    for r0 in (0, 1, rows // 2, rows - 1):
        assert np.array_equal(X.slice(slice(r0, r0 + 1)).to_numpy()[0], exp_row), r0
    s0 = X.sum(0).to_numpy()                              # over the rows: each column sums to rows * value
    assert np.allclose(s0, exp_row.astype(np.float64) * rows, rtol=1e-5)
    s1 = X.sum(1).to_numpy()
    assert np.allclose(s1, float(exp_row.astype(np.float64).sum()), rtol=1e-5)
    X.slice(slice(rows - 1, rows), slice(cols - 1, cols)).copy_from(M.from_numpy(np.array([[100.0]], dtype=np.float32)))
    idx = X.max_axis_idx_ravel(1)                         # per row; the last row's maximum sits past 2^32 elements
    assert idx[-1] == cols - 1 and idx[0] == 6
    print("[exhaustive] 65537 x 65540 elements: ok", flush=True)
