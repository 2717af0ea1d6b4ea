"""Checkpoints in the reference's on-disk formats, for device matrices and optimizer state.

What the reference writes:
  * a Matrix serialises as the struct {shape, stride, data, data_type, ptr_offset}
    (zenu-matrix/src/impl_serde.rs:12-38): `data` is a contiguous row-major copy of the view's
    elements (`new_matrix()`), while `stride` and `ptr_offset` are the view's own -- for a whole
    tensor they are the default stride and 0;
  * a Variable serialises as its data Matrix (zenu-autograd/src/lib.rs:149-160, 320-331);
  * `save_model` (zenu/src/lib.rs:26-37) writes `bincode::serialize(&HashMap<String, Variable>)`;
    `load_model` (:40-67) refuses a file that holds a key the model does not have.

bincode 1.3.3 (zenu/Cargo.toml:22; the crate is not vendored in the reference) with the default
options of `bincode::serialize`: little endian, fixed-width integers, every length and every
`usize` a u64; a struct is its fields in order with no names; a String is a length and UTF-8
bytes; a Vec is a length and its elements; a HashMap is a length and (key, value) pairs in the
map's iteration order, which is arbitrary.  The reference holds no binary fixture, so the byte
layout is pinned by that published format only; the field order, names and value syntax are pinned
by the JSON fixture in impl_serde.rs:242-275, reproduced by `matrix_to_json`.

The reference does not checkpoint its optimizers.  `save_optimizer` / `load_optimizer` write Adam /
AdamW state (m, v per parameter, the step count, the hyper-parameters) as a second file in the same
container, keys `m.<name>`, `v.<name>` and 0-d entries `step`, `learning_rate`, `beta1`, `beta2`,
`epsilon`, `weight_decay`, so that a model file stays loadable by the reference's `load_model`.
"""
import struct

import numpy as np

from .matrix import Matrix, default_stride

_TYPE_NAME = {np.dtype(np.float32): "f32", np.dtype(np.float64): "f64"}
_DTYPE = {v: k for k, v in _TYPE_NAME.items()}


# ---- records: the five serialised fields, on the host ----------------------------------------------

def record_from_numpy(arr):
    """record of a whole (default stride, offset 0) tensor"""
    arr = np.ascontiguousarray(arr) if np.ndim(arr) else np.asarray(arr)
    return {"shape": [int(s) for s in arr.shape], "stride": [int(s) for s in default_stride(arr.shape)],
            "data": arr.reshape(-1).copy(), "data_type": _TYPE_NAME[arr.dtype], "ptr_offset": 0}


def record_from_matrix(m):
    """impl_serde.rs:17-27: contiguous copy of the elements, the view's own stride and offset"""
    data = m.new_matrix().to_numpy().reshape(-1)
    return {"shape": list(m.shape), "stride": list(m.stride), "data": data,
            "data_type": _TYPE_NAME[m.dtype], "ptr_offset": int(m.offset)}


def numpy_from_record(rec):
    """The elements a deserialised Matrix addresses (impl_serde.rs:145-168: pointer = data +
    ptr_offset, then shape and stride as stored)."""
    data = np.asarray(rec["data"], dtype=_DTYPE[rec["data_type"]])
    shape, stride, off = tuple(rec["shape"]), tuple(rec["stride"]), int(rec["ptr_offset"])
    n = int(np.prod(shape, dtype=np.int64)) if shape else 1
    if n == 0:
        return np.zeros(shape, dtype=data.dtype)
    last = off + sum((s - 1) * st for s, st in zip(shape, stride))
    if off < 0 or last >= data.size:
        raise ValueError("shape, stride and ptr_offset address elements outside data")
    isz = data.dtype.itemsize
    view = np.lib.stride_tricks.as_strided(data[off:], shape=shape, strides=tuple(st * isz for st in stride))
    return np.array(view, copy=True, order="C")


def matrix_from_record(rec):
    return Matrix.from_numpy(numpy_from_record(rec))


# ---- bincode 1.3 ---------------------------------------------------------------------------------------

def _u64(v):
    return struct.pack("<Q", int(v))


def _string(s):
    b = s.encode("utf-8")
    return _u64(len(b)) + b


def encode_record(rec):
    data = np.ascontiguousarray(rec["data"], dtype=_DTYPE[rec["data_type"]])
    out = [_u64(len(rec["shape"]))] + [_u64(s) for s in rec["shape"]]
    out += [_u64(len(rec["stride"]))] + [_u64(s) for s in rec["stride"]]
    out += [_u64(data.size), data.astype(data.dtype.newbyteorder("<"), copy=False).tobytes()]
    out += [_string(rec["data_type"]), _u64(rec["ptr_offset"])]
    return b"".join(out)


class _Reader:
    def __init__(self, buf):
        self.buf, self.pos = memoryview(buf), 0

    def take(self, n):
        if n < 0 or self.pos + n > len(self.buf):
            raise ValueError("truncated checkpoint")
        b = self.buf[self.pos:self.pos + n]
        self.pos += n
        return b

    def u64(self):
        return struct.unpack("<Q", self.take(8))[0]

    def string(self):
        return bytes(self.take(self.u64())).decode("utf-8")

    def usizes(self):
        n = self.u64()
        return list(struct.unpack(f"<{n}Q", self.take(8 * n))) if n else []


def decode_record(r, expect_type=None):
    shape, stride = r.usizes(), r.usizes()
    n = r.u64()
    start = r.pos
    # the element width is only known from data_type, which FOLLOWS the data: try both widths
    for name, dt in _DTYPE.items():
        r.pos = start
        try:
            raw = r.take(n * dt.itemsize)
            mark = r.pos
            if r.string() == name:
                data = np.frombuffer(raw, dtype=dt.newbyteorder("<")).astype(dt)
                off = r.u64()
                if expect_type is not None and name != expect_type:
                    raise TypeError("Data type mismatch")          # impl_serde.rs:155-157
                return {"shape": shape, "stride": stride, "data": data, "data_type": name, "ptr_offset": off}
            r.pos = mark
        except (ValueError, UnicodeDecodeError):
            pass
    raise ValueError("not a Matrix record")


def encode_state_dict(records):
    """bincode of HashMap<String, Variable>: records is a mapping name -> record"""
    out = [_u64(len(records))]
    for k, rec in records.items():
        out += [_string(k), encode_record(rec)]
    return b"".join(out)


def decode_state_dict(buf, expect_type=None):
    r = _Reader(buf)
    out = {}
    for _ in range(r.u64()):
        k = r.string()
        out[k] = decode_record(r, expect_type)
    if r.pos != len(r.buf):
        raise ValueError("trailing bytes after the state dict")
    return out


# ---- serde_json (the format the reference's own fixture pins) ------------------------------------------

def _shortest_digits(x, dtype):
    """(digits, exponent) of the shortest decimal that round-trips in dtype: value = 0.d1d2... x 10^exp"""
    s = np.format_float_scientific(dtype.type(x), unique=True, trim="-")
    mant, exp = s.split("e")
    digits = mant.replace("-", "").replace(".", "")
    return digits, int(exp) + 1


def _ryu(x, dtype):
    """Float formatting of serde_json (the ryu crate's `format_finite`): shortest round-trip digits,
    plain notation while the decimal point stays within 16 (f64) / 13 (f32) digits on the left and
    5 / 6 zeros on the right, `e` notation otherwise; non-finite values are `null`."""
    dtype = np.dtype(dtype)
    if not np.isfinite(x):
        return "null"
    sign = "-" if np.signbit(x) else ""
    if x == 0:
        return sign + "0.0"
    digits, kk = _shortest_digits(abs(x), dtype)      # value = 0.DIGITS x 10^kk, kk = position of the point
    n = len(digits)
    wide, small = (16, -5) if dtype == np.float64 else (13, -6)
    if n <= kk <= wide:
        return sign + digits + "0" * (kk - n) + ".0"
    if 0 < kk <= wide:
        return sign + digits[:kk] + "." + digits[kk:]
    if small < kk <= 0:
        return sign + "0." + "0" * (-kk) + digits
    e = kk - 1
    if n == 1:
        return f"{sign}{digits}e{e}"
    return f"{sign}{digits[0]}.{digits[1:]}e{e}"


def matrix_to_json(rec, pretty=True):
    """serde_json::to_string_pretty / to_string of a Matrix (impl_serde.rs:242-275)"""
    dt = _DTYPE[rec["data_type"]]
    if pretty:
        def seq(items):
            items = list(items)
            return "[]" if not items else "[\n" + ",\n".join("    " + i for i in items) + "\n  ]"
        return ("{\n" + f'  "shape": {seq(str(int(s)) for s in rec["shape"])},\n'
                + f'  "stride": {seq(str(int(s)) for s in rec["stride"])},\n'
                + f'  "data": {seq(_ryu(v, dt) for v in rec["data"])},\n'
                + f'  "data_type": "{rec["data_type"]}",\n' + f'  "ptr_offset": {int(rec["ptr_offset"])}\n' + "}")
    j = lambda items: "[" + ",".join(items) + "]"
    return ("{" + f'"shape":{j(str(int(s)) for s in rec["shape"])},"stride":{j(str(int(s)) for s in rec["stride"])},'
            + f'"data":{j(_ryu(v, dt) for v in rec["data"])},"data_type":"{rec["data_type"]}",'
            + f'"ptr_offset":{int(rec["ptr_offset"])}' + "}")


def matrix_from_json(text, expect_type=None):
    import json
    d = json.loads(text)
    for f in ("shape", "stride", "data", "data_type", "ptr_offset"):
        if f not in d:
            raise ValueError(f"missing field `{f}`")
    if expect_type is not None and d["data_type"] != expect_type:
        raise TypeError("Data type mismatch")
    d["data"] = np.asarray([np.nan if v is None else v for v in d["data"]], dtype=_DTYPE[d["data_type"]])
    return d


# ---- models and optimizers ---------------------------------------------------------------------------------

def save_model(parameters, path):
    """save_model, zenu/src/lib.rs:26-37; `parameters`: name -> Matrix (or (Matrix, grad) pairs)"""
    recs = {k: record_from_matrix(v[0] if isinstance(v, tuple) else v) for k, v in parameters.items()}
    with open(path, "wb") as f:
        f.write(encode_state_dict(recs))


def load_model(path, parameters):
    """load_model, zenu/src/lib.rs:40-67: copies every stored tensor into the model's parameter of
    the same name; a stored key the model lacks is an error (before anything is copied here)"""
    with open(path, "rb") as f:
        recs = decode_state_dict(f.read())
    for k in recs:
        if k not in parameters:
            raise KeyError("Failed to load model")
    for k, rec in recs.items():
        dst = parameters[k][0] if isinstance(parameters[k], tuple) else parameters[k]
        dst.copy_from(matrix_from_record(rec))


_HYPER = ("learning_rate", "beta1", "beta2", "epsilon")


def save_optimizer(opt, path):
    """Adam / AdamW state in the same container (no counterpart in the reference)"""
    recs = {}
    for k, m in opt.m.items():
        recs[f"m.{k}"] = record_from_matrix(m)
        recs[f"v.{k}"] = record_from_matrix(opt.v[k])
    scalars = {h: getattr(opt, h) for h in _HYPER}
    scalars["step"] = opt.step
    if hasattr(opt, "weight_decay"):
        scalars["weight_decay"] = opt.weight_decay
    for k, v in scalars.items():
        recs[k] = record_from_numpy(np.asarray(v, dtype=np.float64))
    with open(path, "wb") as f:
        f.write(encode_state_dict(recs))


def load_optimizer(path, opt):
    with open(path, "rb") as f:
        recs = decode_state_dict(f.read())
    for k, rec in recs.items():
        if k.startswith("m.") or k.startswith("v."):
            table = opt.m if k[0] == "m" else opt.v
            if k[2:] not in table:
                raise KeyError("Failed to load optimizer")
    for k, rec in recs.items():
        if k.startswith("m.") or k.startswith("v."):
            (opt.m if k[0] == "m" else opt.v)[k[2:]].copy_from(matrix_from_record(rec))
        elif k == "step":
            opt.step = type(opt.step)(numpy_from_record(rec))
        elif k in _HYPER or k == "weight_decay":
            setattr(opt, k, float(numpy_from_record(rec)))
