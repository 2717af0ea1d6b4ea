"""Pins the CPU oracle against the reference's own known-answer tests (CPU only)."""
import numpy as np
import pytest

import cpu_matrix
import ref_cases
import zenu_oracle as zo


class CpuDev:
    M = cpu_matrix.CpuMatrix
    sum_to = staticmethod(cpu_matrix.sum_to)
    F = cpu_matrix
    Error = (zo.OracleError, Exception)


@pytest.mark.parametrize("case", ref_cases.CASES, ids=lambda c: c.__name__)
def test_oracle_ref_case(case):
    case(CpuDev)


def test_leaf_call_counts():
    """with_clousers.rs:356-379: a default-stride [10,10,10] operand is ONE leaf call, the
    `.., ..;2, ..` slice is 50 (10 x 5 rows)."""
    a = np.zeros((10, 10, 10), dtype=np.float32)
    zo.reset_leaf_calls()
    zo.binary_scalar_assign(zo.ADD, a, 1.0)
    assert zo.leaf_calls() == 1
    zo.reset_leaf_calls()
    zo.binary_scalar_assign(zo.ADD, a[:, ::2, :], 1.0)
    assert zo.leaf_calls() == 50
    # the BASELINE shapes: row-broadcast and transposed adds are one leaf call per row
    x = np.zeros((64, 32), dtype=np.float32)
    out = np.zeros_like(x)
    zo.reset_leaf_calls()
    zo.binary_array(zo.ADD, out, x, np.zeros((1, 32), dtype=np.float32))
    assert zo.leaf_calls() == 64
    zo.reset_leaf_calls()
    zo.binary_array(zo.ADD, out, x, np.zeros((32, 64), dtype=np.float32).T)
    assert zo.leaf_calls() == 64
    zo.reset_leaf_calls()
    zo.unary(zo.EXP, out, x)  # unary always recurses to 1-D (basic_operations.rs:529-535)
    assert zo.leaf_calls() == 64
    zo.reset_leaf_calls()
    zo.sum_axis(x, 0)         # shape[axis] slice adds (sum.rs:20-25)
    assert zo.leaf_calls() == 64


def test_unary_range_hash_is_the_fold_of_the_element_wise_results():
    """zo.unary_range_hash (the host side of the every-argument comparison with the device): a block's sum
    is the sum of the documented term over the element-wise results of the same function, NaN results
    count as one value, threads only split the blocks, and the sigmoid composite is zo.sigmoid"""
    def fold(bits, res):
        rb = res.view(np.uint32).astype(np.uint64)
        rb = np.where(np.isnan(res), np.uint64(0x7fc00000), rb)
        z = (bits.astype(np.uint64) << np.uint64(32)) | rb
        with np.errstate(over="ignore"):
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xbf58476d1ce4e5b9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94d049bb133111eb)
            z = z ^ (z >> np.uint64(31))
            return int(z.sum(dtype=np.uint64))
    for fn, first in ((zo.TANH, 0x3f000000), (zo.EXP, 0xc2000000), (zo.LOG, 0xbf7f0000), (zo.SIGMOID_COMPOSITE, 0x7f7f0000),
                      (zo.ASIN, 0x3f7f0000)):
        sums = zo.unary_range_hash(fn, first, 4 << 16, 16, 3)
        assert np.array_equal(sums, zo.unary_range_hash(fn, first, 4 << 16, 16, 1))
        for b in range(4):
            bits = np.arange(first + (b << 16), first + ((b + 1) << 16), dtype=np.uint64).astype(np.uint32)
            x = bits.view(np.float32)
            out = np.empty_like(x)
            with np.errstate(all="ignore"):
                zo.sigmoid(out, x) if fn == zo.SIGMOID_COMPOSITE else zo.unary(fn, out, x)
            assert fold(bits, out) == int(sums[b]), (fn, b)
    assert zo.range_hash_term(1, 0x7fc00001) == zo.range_hash_term(1, 0xffc12345)     # any NaN
    assert zo.range_hash_term(1, 2) != zo.range_hash_term(2, 1)
    with pytest.raises(zo.OracleError):
        zo.unary_range_hash(zo.TANH, 0, (1 << 16) + 5, 16, 1)


def test_powf_and_f64_range_hashes_are_folds_of_the_element_wise_results():
    """the powf and f64 forms of the host-side fold: a block's sum equals the sum of the documented terms over
    element-wise results, the f64 arguments are the documented (high word, pseudo-random low word) pairs"""
    def mix(z):
        with np.errstate(over="ignore"):
            z = (z ^ (z >> np.uint64(30))) * np.uint64(0xbf58476d1ce4e5b9)
            z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94d049bb133111eb)
            return z ^ (z >> np.uint64(31))
    first = 0xbf000000            # negative bases: NaN results
    sums = zo.powf_range_hash(np.float32(2.5), first, 2 << 16, 16, 2)
    for b in range(2):
        bits = np.arange(first + (b << 16), first + ((b + 1) << 16), dtype=np.uint64).astype(np.uint32)
        x = bits.view(np.float32)
        out = np.empty_like(x)
        with np.errstate(all="ignore"):
            zo.powf(out, x, 2.5)
        rb = np.where(np.isnan(out), np.uint64(0x7fc00000), out.view(np.uint32).astype(np.uint64))
        with np.errstate(over="ignore"):
            assert int(mix((bits.astype(np.uint64) << np.uint64(32)) | rb).sum(dtype=np.uint64)) == int(sums[b])
    step, offset, salt = 4, 3, 7
    i0 = 0x0ff00000               # high words around 0x3fc00000: arguments near 0.125 .. 
    sums = zo.unary_range_hash_f64(zo.TANH, i0, 2 << 12, 12, step, offset, salt, 2)
    for b in range(2):
        idx = np.arange(i0 + (b << 12), i0 + ((b + 1) << 12), dtype=np.uint64)
        with np.errstate(over="ignore"):
            hi = (idx * np.uint64(step) + np.uint64(offset)) & np.uint64(0xffffffff)
            lo = (((idx + np.uint64(salt)) * np.uint64(0x9E3779B97F4A7C15)) >> np.uint64(29)) & np.uint64(0xffffffff)
        bits = (hi << np.uint64(32)) | lo
        assert int(bits[5]) == zo.range_arg_f64(int(idx[5]), step, offset, salt)
        x = bits.view(np.float64)
        out = np.empty_like(x)
        zo.unary(zo.TANH, out, x)
        rb = np.where(np.isnan(out), np.uint64(0x7ff8000000000000), out.view(np.uint64))
        with np.errstate(over="ignore"):
            assert int(mix(mix(bits) + rb).sum(dtype=np.uint64)) == int(sums[b])
    # the f64 powf over the same arguments
    sums = zo.powf_range_hash_f64(-1.5, i0, 2 << 12, 12, step, offset, salt, 2)
    for b in range(2):
        idx = np.arange(i0 + (b << 12), i0 + ((b + 1) << 12), dtype=np.uint64)
        with np.errstate(over="ignore"):
            hi = (idx * np.uint64(step) + np.uint64(offset)) & np.uint64(0xffffffff)
            lo = (((idx + np.uint64(salt)) * np.uint64(0x9E3779B97F4A7C15)) >> np.uint64(29)) & np.uint64(0xffffffff)
        bits = (hi << np.uint64(32)) | lo
        x = bits.view(np.float64)
        out = np.empty_like(x)
        with np.errstate(all="ignore"):
            zo.powf(out, x, -1.5)
        rb = np.where(np.isnan(out), np.uint64(0x7ff8000000000000), out.view(np.uint64))
        with np.errstate(over="ignore"):
            assert int(mix(mix(bits) + rb).sum(dtype=np.uint64)) == int(sums[b])
    with pytest.raises(zo.OracleError):
        zo.unary_range_hash_f64(zo.TANH, 0, 1 << 12, 12, 0, 0, 0, 1)
    with pytest.raises(zo.OracleError):
        zo.powf_range_hash_f64(2.0, 0, 1 << 12, 12, 0, 0, 0, 1)
