"""The C++ host API (include/zenu_hip.hpp): the reference's known-answer cases written in C++
(tests/native/cpp_api_check.cpp).  CPU: the program compiles and links against the library with a plain
g++.  GPU: the prebuilt program (built by __graft_entry__.build()) runs every case."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CASES = ["scalar_add_2d", "sliced_3d", "sliced_3d_assign", "matrix_add_sliced", "transposed", "broadcast_add",
         "broadcast_add_1x4x1x1_3x4x5x5", "sub_mul_div", "shape_errors", "unary_tables", "relu_cases", "sigmoid_cases",
         "sum_4d", "max_cases", "asum_cases", "copy_cases", "broadcast_cases", "conv_bias_cases", "mean_variance_cases", "stack_split_cases", "softmax_cases", "cross_entropy_cases",
         "clip_cases", "sgd_net_test", "adam_net_test", "adam_w_net_test", "adam_w_net_test_scheduled"]


def test_cpp_api_program_builds(tmp_path):
    import __graft_entry__ as g
    exe = g.build_cpp_api_check(str(tmp_path / "cpp_api_check"))
    assert os.path.exists(exe)


@pytest.mark.gpu
def test_cpp_api_reference_cases():
    exe = os.path.join(ROOT, "tests", "native", "bin", "cpp_api_check")
    if not os.path.exists(exe):
        pytest.skip("tests/native/bin/cpp_api_check is not built (run __graft_entry__.build())")
    out = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(out.stdout[-3000:], flush=True)
    assert out.returncode == 0, out.stdout + out.stderr
    for name in CASES:
        assert f"ok {name}" in out.stdout, name
