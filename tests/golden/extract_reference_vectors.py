"""Extracts the literal test vectors of the reference's max_axis tests into JSON fixtures.

Run in the build container only (the reference tree is not present on the GPU box):
    python tests/golden/extract_reference_vectors.py
Reads zenu-matrix/src/operation/max.rs as TEXT (the Rust sources cannot be compiled here) and
writes inputs and expected outputs -- data only -- to tests/golden/max_axis_4d_{f32,f64}.json.
Source: max_axis_4d (max.rs:247-545, f32) and max_axis_4d_f64 (max.rs:546-844).
"""
import json
import os
import re

REF = "/root/reference/zenu-matrix/src/operation/max.rs"
HERE = os.path.dirname(os.path.abspath(__file__))


def vec_after(text, name, start):
    m = re.compile(r"let\s+" + name + r"(?:\s*:\s*Vec<f(?:32|64)>)?\s*=\s*vec!\[(.*?)\];", re.S).search(text, start)
    nums = [float(x) for x in re.findall(r"-?\d+\.\d+(?:e-?\d+)?|-?\d+", m.group(1))]
    return nums, m.end()


def extract(fn_name, out_name):
    text = open(REF).read()
    start = text.index("fn " + fn_name + "<D: Device>()")
    data = {"source": f"zenu-matrix/src/operation/max.rs fn {fn_name}", "shape": [2, 3, 4, 5]}
    pos = start
    for key in ("input", "ans_0d", "ans_1d", "ans_2d", "ans_3d"):
        data[key], pos = vec_after(text, key, pos)
    assert len(data["input"]) == 120 and len(data["ans_0d"]) == 60 and len(data["ans_1d"]) == 40
    assert len(data["ans_2d"]) == 30 and len(data["ans_3d"]) == 24
    with open(os.path.join(HERE, out_name), "w") as f:
        json.dump(data, f, indent=0)


if __name__ == "__main__":
    extract("max_axis_4d", "max_axis_4d_f32.json")
    text = open(REF).read()
    names = re.findall(r"fn (max_axis_4d\w*)<D: Device>", text)
    for n in names:
        if n != "max_axis_4d":
            extract(n, "max_axis_4d_f64.json")
    print("wrote fixtures for", names)
