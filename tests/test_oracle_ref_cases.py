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
