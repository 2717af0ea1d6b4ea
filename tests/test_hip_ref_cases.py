"""The reference's known-answer tests on the HIP device (the `_gpu` leg of run_mat_test!)."""
import pytest

import ref_cases

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hipdev(hip):
    class HipDev:
        M = hip.Matrix
        sum_to = staticmethod(hip.sum_to)
        F = hip
        Error = hip.ZenuHipError
    return HipDev


@pytest.mark.parametrize("case", ref_cases.CASES, ids=lambda c: c.__name__)
def test_hip_ref_case(case, hipdev):
    print(f"[case] {case.__name__}", flush=True)
    case(hipdev)
