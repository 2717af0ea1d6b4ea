"""CPU-only checks of the host-side native code: the allocator's bookkeeping against a fake device
backend, and the device math header compiled for the host against the host libm."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NATIVE = os.path.join(ROOT, "tests", "native")


def build(src, out, extra=()):
    cmd = ["g++", "-O2", "-std=c++17", "-Wall", *extra, "-o", out, os.path.join(NATIVE, src), "-lpthread", "-lm"]
    subprocess.check_call(cmd)
    return out


def test_allocator_bookkeeping(tmp_path):
    """mirrors zenu-matrix/src/memory_pool/test.rs:51-422 (mock device) for the new allocator:
    size classes, same-stream and cross-stream reuse, split/merge, OOM -> trim -> retry, foreign
    pointers, blocks taken during a stream capture staying out of ordinary requests until released,
    and a randomized stress run against a shadow model"""
    exe = build("allocator_host_check.cpp", str(tmp_path / "alloc_check"),
                ("-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined"))   # the bookkeeping under the sanitizers
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    for name in ("size_classes", "same_stream_reuse", "cross_stream_reuse", "retire_stream", "split_merge_trim", "oom_retry",
                 "injected_failure", "not_owned", "capture_blocks", "stress"):
        assert f"ok {name}" in out.stdout


def test_shape_algebra_against_brute_force(tmp_path):
    """zenu_amd/csrc/shape.cpp compiled for the host (address and undefined-behaviour sanitizers on): 20 000
    seeded random elementwise problems -- up to six dims, three operands, permuted / sliced / broadcast
    strides -- must visit exactly the original (output, input, input) offsets after ew_collapse, with no
    size-1 dim left and the output's strides in decreasing order; the alias rule must refuse every pair of
    views that share an element without being the same view, accept the output's own view and every pair of
    disjoint ranges (60 000 random pairs against an element-by-element model); the shape rules on the
    reference's own cases (dim_dyn.rs:24-58, broadcast.rs:13-44)"""
    exe = build("shape_host_check.cpp", str(tmp_path / "shape_check"),
                ("-g", "-O1", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include", "-fsanitize=address,undefined",
                 "-fno-sanitize-recover=undefined"))
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    for name in ("collapse", "alias", "rules"):
        assert f"ok {name}" in out.stdout


def test_zmath_matches_host_libm(tmp_path):
    """zmath.hpp (the transcendental functions the kernels use) compiled for the host with
    contraction off must give the bits of the host libm: f32 tanh, expm1, exp, log, sinh, cosh (both forms), sin,
    cos, tan, atan, asin, acos and the sigmoid composite on every 31st f32 bit pattern (138 M points
    each; stride 1, all 2^32, was run during development with the same result); powf on every 31st
    base for 19 fixed exponents and on two pseudo-random (base, exponent) pairs per base; f64 tanh,
    expm1, exp, log, sinh, cosh and the sigmoid composite on every 31st high word with three low words
    each plus uniform samples in +-745 and +-4 (about 700 M points); f64 pow in both of its forms on 5 * 10^7 pairs
    (uniform bit patterns for both arguments, moderate pairs, negative and log-uniform bases under 22 fixed
    exponents); f64 sin and cos on every 248th high
    word with three low words each plus uniform samples in each of their six argument ranges (150 M points each); f64 tanh in both of its forms
    (fdlibm's branches and the single path the kernels use) and the sigmoid also on 400 M uniform
    samples in +-1, +-4 and +-20.  tanhf_ulp2, the variant that
    is not meant to give libm's bits, must stay within 2 units in the last place of tanhf on the
    same f32 points (stride 1: the largest distance is 2)."""
    exe = build("zmath_host_check.cpp", str(tmp_path / "zmath_check"), ("-ffp-contract=off", "-fno-fast-math"))
    out = subprocess.run([exe, "31"], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout
    assert out.stdout.split() == ["tanhf_fdlibm", "0", "tanhf_simd", "0", "expm1f_fdlibm", "0", "sigmoidf_zenu", "0",
                                  "tanh_fdlibm", "0", "expm1_fdlibm", "0", "sigmoid_zenu", "0",
                                  "exp_glibc", "0", "sinh_fdlibm", "0", "cosh_fdlibm", "0",
                                  "expf_glibc", "0", "logf_glibc", "0", "powf_glibc", "0",
                                  "sinhf_fdlibm", "0", "coshf_fdlibm", "0", "sinhf_simd", "0", "coshf_simd", "0", "sinf_glibc", "0", "cosf_glibc", "0",
                                  "atanf_fdlibm", "0", "asinf_fdlibm", "0", "acosf_fdlibm", "0",
                                  "tanhf_ulp2_beyond_2ulp", "0", "tanf_glibc", "0", "sin_glibc", "0", "cos_glibc", "0", "log_glibc", "0", "pow_glibc", "0"]


def _macro_numbers(text, name, following, pattern):
    import re
    start = text.index("#define " + name)
    return re.findall(pattern, text[start:text.index(following, start)])


def test_generated_tables_are_what_their_generators_give(tmp_path):
    """the tables of the f64 sine / cosine and the f64 log in zmath.hpp against the programs that make them:
    sin(k/128), cos(k/128) and the pieces of 2/pi in full; of the log table (two and a half minutes of search
    for all 128 subintervals) the first two subintervals and the last, where the host libm picks the entry
    among the candidates of the published construction; the log table of the f64 pow in full"""
    import re
    import sys
    src = open(os.path.join(ROOT, "zenu_amd", "csrc", "zmath.hpp")).read()
    gen_dir = os.path.join(ROOT, "zenu_amd", "csrc", "tablegen")
    out = subprocess.run([sys.executable, os.path.join(gen_dir, "sincos64_tables.py")], capture_output=True, text=True, check=True).stdout
    sincos, toverp = out.split("ZM_TOVERP_TAB")
    hexes = r"0x[0-9a-f]{16}ull"
    assert re.findall(hexes, sincos) == _macro_numbers(src, "ZM_SINCOS64_TAB", "#define ZM_TOVERP_TAB", hexes)
    assert re.findall(r"\d+\.0", toverp) == _macro_numbers(src, "ZM_TOVERP_TAB", "static const uint64_t kSinCos64TabHost", r"\d+\.0")
    out = subprocess.run([sys.executable, os.path.join(gen_dir, "pow64_table.py")], capture_output=True, text=True, check=True).stdout
    assert re.findall(hexes, out) == _macro_numbers(src, "ZM_POW64_LOG_TAB", "static const uint64_t kPow64LogTabHost", hexes)
    exe = str(tmp_path / "log64_table")
    subprocess.check_call(["g++", "-O2", "-std=gnu++17", "-fext-numeric-literals", "-ffp-contract=off", "-mfma", "-fopenmp",
                           os.path.join(gen_dir, "log64_table.cpp"), "-lquadmath", "-o", exe])
    table = _macro_numbers(src, "ZM_LOG64_TAB", "static const uint64_t kLog64TabHost", hexes)
    assert len(table) == 256
    for first, last in ((0, 2), (127, 128)):
        got = subprocess.run([exe, str(first), str(last)], capture_output=True, text=True)
        assert got.returncode == 0, got.stderr
        assert re.findall(hexes, got.stdout) == table[2 * first:2 * last]
