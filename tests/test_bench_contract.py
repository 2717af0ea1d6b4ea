"""bench.py's command line and its one JSON line: the keys the driver reads, the roofline and cpu_baseline
objects, the refusal of more than one GPU.  The CPU part needs no GPU (the refusal comes before anything
touches the device); the GPU part runs a short configs[0] pass."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args, timeout=300):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=timeout, cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    out = run_bench("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert out.returncode != 0
    assert "ONE GPU" in (out.stderr + out.stdout)
    assert not out.stdout.strip().startswith("{")          # no JSON line that could be mistaken for a result


@pytest.mark.gpu
def test_json_line_has_the_contract_keys():
    out = run_bench("--workload", "c0", "--steps", "3", "--warmup", "1", "--op-reps", "5")
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [l for l in out.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "ops"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 3 and d["warmup"] == 1
    assert d["unit"] == "GB/s" and d["higher_is_better"] is True and d["vs_baseline"] is None
    assert d["data"] == "synthetic" and "workload" in d["config"] and "model" not in d["config"]
    assert 0 < d["value"] < 8000.0 and d["ms_per_step"] > 0
    r = d["roofline"]
    assert r["bound"] == "hbm" and r["unit"] == "GB/s" and r["peak"] == 8000.0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3 and 0 < r["frac"] < 1
    assert "traffic" in r
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] == 1 and c["unit"] == "GB/s" and c["value"] > 0 and c["sample"]
    ops = {o["op"]: o for o in d["ops"]}
    assert set(ops) == {"add[2^24]", "mul[2^24]", "relu[2^24]", "copy[2^24]"}
    for o in ops.values():
        assert len(o["us_batches"]) == 3 and sorted(o["us_batches"])[1] == o["us"]
        assert 0 < o["frac_of_peak"] < 1
