"""bindings/zenu_hip_sys.rs (the Rust FFI declarations a zenu-hip-kernel-sys crate would hold, in
place of the bindgen output of zenu-cuda-kernel-sys/build.rs:35-53) is generated from
include/zenu_hip.h.  Regenerate it and compare, and check it independently against the header's
symbol list and the ctypes signature table, so neither the .rs file nor the excerpt shown in
the binder's guide at the repository root can drift from the header.  The file itself was never compiled (no Rust here)."""
import ctypes as C
import importlib.util
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _generator():
    spec = importlib.util.spec_from_file_location("gen_rust_bindings", os.path.join(ROOT, "bindings", "gen_rust_bindings.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _functions(text):
    """name -> (list of argument types, return type or None) from the extern block"""
    out = {}
    for m in re.finditer(r"pub fn (\w+)\((.*?)\)( -> ([^;]+))?;", text):
        args = [a.split(":", 1)[1].strip() for a in m.group(2).split(", ")] if m.group(2).strip() else []
        out[m.group(1)] = (args, m.group(4))
    return out


def test_generated_file_is_current():
    gen = _generator()
    assert open(gen.OUT).read() == gen.generate(), "run python bindings/gen_rust_bindings.py"


def test_every_declared_symbol_is_bound_with_matching_arity_and_types():
    from test_c_abi_exports import declared_symbols
    from zenu_amd import _lib
    fns = _functions(open(os.path.join(ROOT, "bindings", "zenu_hip_sys.rs")).read())
    declared = declared_symbols()
    assert sorted(fns) == sorted(declared)                     # nothing missing, nothing extra
    # zenu_hip_* entry points: the ctypes table is a second, hand-written reading of the header
    # (on LP64, ctypes' c_size_t and c_uint64 are one class: a size_t parameter reads usize, a uint64_t one u64)
    ctypes_to_rust = {C.c_int: {"c_int"}, C.c_int64: {"i64"}, C.c_double: {"f64"}, C.c_size_t: {"usize", "u64"}, C.c_uint32: {"u32"}}
    for name, argtypes in _lib.SIGNATURES.items():
        rargs, ret = fns[name]
        assert len(rargs) == len(argtypes), name
        assert ret == "c_int", name
        for ra, ca in zip(rargs, argtypes):
            if ca in ctypes_to_rust:
                assert ra in ctypes_to_rust[ca], (name, ra, ca)
            elif ca is C.c_void_p:
                assert ra == "ZenuStream" or ra.startswith("*"), (name, ra)
            else:                                              # POINTER(...)
                assert ra.startswith("*"), (name, ra)
                if getattr(ca, "_type_", None) is _lib.Tensor:
                    assert ra == "*const ZenuTensor", (name, ra)
    assert fns["zenu_hip_status_string"] == (["c_int"], "*const c_char")
    # the reference-named functions return nothing and take the element type of their suffix
    ref = _lib.reference_named_symbols()
    assert len(ref) == 126
    for name in ref:
        rargs, ret = fns[name]
        assert ret is None, name
        ty = "f32" if name.endswith("_float") else "f64"
        ptrs = [a for a in rargs if a.startswith("*")]
        assert ptrs and all(a in (f"*mut {ty}", f"*const {ty}", "*mut c_int") for a in ptrs), (name, rargs)
    assert fns["array_array_add_float"][0] == ["*mut f32", "c_int", "*mut f32", "c_int", "*mut f32", "c_int", "c_int"]
    assert fns["relu_double"][0] == ["*mut f64", "*mut f64", "f64", "c_int", "c_int", "c_int"]


def test_struct_layout_matches_the_ctypes_mirror():
    from zenu_amd import _lib
    text = open(os.path.join(ROOT, "bindings", "zenu_hip_sys.rs")).read()
    m = re.search(r"pub struct ZenuTensor \{(.*?)\}", text, re.S)
    fields = [tuple(x.strip() for x in f.replace("pub ", "").split(":")) for f in m.group(1).strip().rstrip(",").split(",\n")]
    assert fields == [("ptr", "*mut c_void"), ("ndim", "i32"), ("reserved", "i32"),
                      ("shape", "[i64; ZENU_MAX_DIM]"), ("stride", "[i64; ZENU_MAX_DIM]")]
    assert [n for n, _ in _lib.Tensor._fields_] == [n for n, _ in fields]
    assert C.sizeof(_lib.Tensor) == 8 + 4 + 4 + 2 * 6 * 8
    m = re.search(r"pub struct ZenuMempoolStats \{(.*?)\}", text, re.S)
    names = re.findall(r"pub (\w+): u64", m.group(1))
    assert names == [n for n, _ in _lib.MempoolStats._fields_]
    for k, v in (("ZENU_ERR_SCRATCH_LIMIT", _lib.ERR_SCRATCH_LIMIT), ("ZENU_TANH_ULP2", _lib.TANH_ULP2), ("ZENU_F64", _lib.F64)):
        assert re.search(rf"pub const {k}: c_int = {v};", text)


def test_integration_excerpt_is_taken_from_the_generated_file():
    """every `pub fn` line the binder's guide shows must be a line of the generated file"""
    doc = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    gen = open(os.path.join(ROOT, "bindings", "zenu_hip_sys.rs")).read()
    shown = re.findall(r"^\s*(pub fn \w+\(.*\).*;)\s*$", doc, re.M)
    assert shown, "the guide shows no binding lines"
    for line in shown:
        assert line in gen, line
