"""Checkpoint formats (zenu_amd/checkpoint.py): the reference's JSON fixture, the bincode container,
and -- on the GPU -- device round trips and an optimizer resume.

Pinned by: the pretty-JSON literal of zenu-matrix/src/impl_serde.rs:242-275 (field order, names,
number syntax), its type-mismatch test (:277-289), known outputs of Rust's shortest round-trip
float printing, and a byte string written out by hand from bincode 1.3's published layout.
"""
import struct

import numpy as np
import pytest

from zenu_amd import checkpoint as ck


def test_json_fixture_of_the_reference():
    rec = ck.record_from_numpy(np.array([[1., 2.], [3., 4.]], dtype=np.float32))
    expected = """{
  "shape": [
    2,
    2
  ],
  "stride": [
    2,
    1
  ],
  "data": [
    1.0,
    2.0,
    3.0,
    4.0
  ],
  "data_type": "f32",
  "ptr_offset": 0
}"""
    assert ck.matrix_to_json(rec) == expected
    back = ck.matrix_from_json(expected, "f32")
    assert np.array_equal(ck.numpy_from_record(back), [[1, 2], [3, 4]])
    assert ck.matrix_to_json(ck.matrix_from_json(ck.matrix_to_json(rec, pretty=False))) == expected


def test_json_type_mismatch_is_an_error():   # impl_serde.rs:277-289
    bad = '{"shape": [2, 2], "stride": [2, 1], "data": [1.0, 2.0, 3.0, 4.0], "data_type": "f64", "ptr_offset": 0}'
    with pytest.raises(TypeError):
        ck.matrix_from_json(bad, "f32")
    with pytest.raises(ValueError):
        ck.matrix_from_json('{"shape": [1], "stride": [1], "data": [1.0], "data_type": "f32"}')


@pytest.mark.parametrize("value,dtype,text", [
    (1.0, np.float64, "1.0"), (0.1, np.float32, "0.1"), (0.1, np.float64, "0.1"), (-2.5, np.float32, "-2.5"),
    (1e15, np.float64, "1000000000000000.0"), (1e16, np.float64, "1e16"), (1.5e16, np.float64, "1.5e16"),
    (123456789012345680.0, np.float64, "1.2345678901234568e17"), (1e-5, np.float64, "0.00001"),
    (1e-6, np.float64, "1e-6"), (1.5e-7, np.float64, "1.5e-7"), (1e30, np.float64, "1e30"),
    (16777216.0, np.float32, "16777216.0"), (1e13, np.float32, "1e13"), (1e12, np.float32, "1000000000000.0"),
    (1e-6, np.float32, "0.000001"), (1e-7, np.float32, "1e-7"), (3.4028235e38, np.float32, "3.4028235e38"),
    (0.0, np.float32, "0.0"), (-0.0, np.float64, "-0.0"), (np.nan, np.float32, "null"), (np.inf, np.float64, "null"),
    (5e-324, np.float64, "5e-324"), (1.17549435e-38, np.float32, "1.1754944e-38"),
])
def test_float_printing_like_rust(value, dtype, text):
    assert ck._ryu(dtype(value), dtype) == text
    if text != "null":
        assert dtype(float(text)) == dtype(value) or (value == 0)


def test_bincode_bytes_by_hand():
    """HashMap{"w": Matrix f32 [2,1] = (1.5, -2)} in bincode 1.3 defaults, written out field by field"""
    u = lambda v: struct.pack("<Q", v)
    by_hand = (u(1)                                  # one entry
               + u(1) + b"w"                         # key
               + u(2) + u(2) + u(1)                  # shape [2, 1]
               + u(2) + u(1) + u(1)                  # stride [1, 1]
               + u(2) + struct.pack("<ff", 1.5, -2.0)   # data
               + u(3) + b"f32"                       # data_type
               + u(0))                               # ptr_offset
    rec = ck.record_from_numpy(np.array([[1.5], [-2.0]], dtype=np.float32))
    assert ck.encode_state_dict({"w": rec}) == by_hand
    back = ck.decode_state_dict(by_hand)
    assert list(back) == ["w"] and back["w"]["data_type"] == "f32" and back["w"]["shape"] == [2, 1]
    assert np.array_equal(ck.numpy_from_record(back["w"]), [[1.5], [-2.0]])


def test_bincode_round_trip_and_errors():
    r = np.random.default_rng(0)
    recs = {"linear1.weight": ck.record_from_numpy(r.standard_normal((5, 7)).astype(np.float32)),
            "linear1.bias": ck.record_from_numpy(r.standard_normal(5).astype(np.float64)),
            "scalar": ck.record_from_numpy(np.float32(3.25)),
            "empty": ck.record_from_numpy(np.zeros((0, 3), dtype=np.float32))}
    blob = ck.encode_state_dict(recs)
    back = ck.decode_state_dict(blob)
    assert set(back) == set(recs)
    for k in recs:
        assert back[k]["data_type"] == recs[k]["data_type"] and back[k]["shape"] == recs[k]["shape"]
        assert np.array_equal(back[k]["data"], recs[k]["data"])
        assert ck.numpy_from_record(back[k]).shape == tuple(recs[k]["shape"])
    with pytest.raises(ValueError):
        ck.decode_state_dict(blob[:-3])
    with pytest.raises(ValueError):
        ck.decode_state_dict(blob + b"\0")
    with pytest.raises(TypeError):
        ck.decode_state_dict(blob, expect_type="f32")
    # a record whose stride / offset point outside its data is refused, not read
    bad = dict(recs["linear1.weight"], stride=[70, 1])
    with pytest.raises(ValueError):
        ck.numpy_from_record(bad)


def test_view_record_semantics():
    """impl_serde.rs:17-27: data is the view's elements in row-major order, stride and ptr_offset stay the
    view's; reading such a record back applies them to the compact data (as the reference does)"""
    rec = {"shape": [2, 3], "stride": [1, 2], "data": np.arange(6, dtype=np.float32), "data_type": "f32", "ptr_offset": 0}
    assert np.array_equal(ck.numpy_from_record(rec), [[0, 2, 4], [1, 3, 5]])


@pytest.mark.gpu
def test_device_round_trip_and_model_files(hip, tmp_path):
    r = np.random.default_rng(1)
    w = r.standard_normal((6, 4)).astype(np.float32)
    b = r.standard_normal(6).astype(np.float64)
    params = {"l.weight": hip.Matrix.from_numpy(w), "l.bias": hip.Matrix.from_numpy(b)}
    path = tmp_path / "model.bin"
    ck.save_model(params, path)
    fresh = {"l.weight": hip.Matrix.zeros((6, 4)), "l.bias": hip.Matrix.zeros((6,), np.float64),
             "other": hip.Matrix.zeros((2,))}
    ck.load_model(path, fresh)
    assert np.array_equal(fresh["l.weight"].to_numpy(), w) and np.array_equal(fresh["l.bias"].to_numpy(), b)
    with pytest.raises(KeyError):                      # zenu/src/lib.rs:62-64
        ck.load_model(path, {"l.weight": fresh["l.weight"]})
    # a transposed view: compact data, the view's stride
    rec = ck.record_from_matrix(params["l.weight"].transpose())
    assert rec["shape"] == [4, 6] and rec["stride"] == [1, 4]
    assert np.array_equal(rec["data"], w.T.reshape(-1))


@pytest.mark.gpu
def test_adam_resume_is_bit_identical(hip, tmp_path):
    r = np.random.default_rng(2)
    p0 = {"a": r.standard_normal((33, 17)).astype(np.float32), "b": r.standard_normal(129).astype(np.float32)}
    grads = [{k: r.standard_normal(v.shape).astype(np.float32) for k, v in p0.items()} for _ in range(6)]

    def run(n_first, resume):
        params = {k: hip.Matrix.from_numpy(v) for k, v in p0.items()}
        opt = hip.AdamW(1e-3, 0.9, 0.999, 1e-8, 0.01, {k: (v, None) for k, v in params.items()}, weights={"a"})
        for g in grads[:n_first]:
            opt.update({k: (params[k], hip.Matrix.from_numpy(g[k])) for k in params})
        if resume:
            ck.save_model(params, tmp_path / "m.bin")
            ck.save_optimizer(opt, tmp_path / "o.bin")
            params = {k: hip.Matrix.zeros(v.shape) for k, v in p0.items()}
            opt = hip.AdamW(0.5, 0.5, 0.5, 0.5, 0.5, {k: (v, None) for k, v in params.items()}, weights={"a"})
            ck.load_model(tmp_path / "m.bin", params)
            ck.load_optimizer(tmp_path / "o.bin", opt)
        for g in grads[n_first:]:
            opt.update({k: (params[k], hip.Matrix.from_numpy(g[k])) for k in params})
        return {k: v.to_numpy() for k, v in params.items()}

    straight, resumed = run(6, False), run(3, True)
    for k in p0:
        assert np.array_equal(straight[k].view(np.uint32), resumed[k].view(np.uint32)), k
