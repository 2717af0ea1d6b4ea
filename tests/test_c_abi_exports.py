"""The C-ABI library loads without a GPU and exports every symbol include/zenu_hip.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "zenu_hip.h")).read()
    macro = re.search(r"#define ZENU_DECL_1D\(T, S\)(.*?)\n\nZENU_DECL_1D", text, re.S).group(1)
    plain = re.sub(r"#define ZENU_DECL_1D.*?\n\n", "", text, flags=re.S)
    names = set(re.findall(r"\b(?:int|const char \*)\s*(zenu_hip_\w+)\s*\(", plain))
    for tmpl in re.findall(r"\bvoid\s+(\w+)##S\s*\(", macro):
        for s in ("float", "double"):
            names.add(tmpl + s)
    return sorted(names)


def test_header_is_parsed():
    names = declared_symbols()
    assert "zenu_hip_binary" in names and "zenu_hip_adam_step_multi" in names
    assert "array_array_add_float" in names and "memory_set_double" in names
    assert len(names) >= 40 + 2 * 40


def test_library_exports_every_declared_symbol():
    import zenu_amd
    lib = zenu_amd.lib()                      # raises if the shared object is missing
    missing = [n for n in declared_symbols() if not hasattr(lib, n)]
    assert not missing, missing
    from zenu_amd import _lib
    assert not [n for n in _lib.SIGNATURES if not hasattr(lib, n)]
    ref = _lib.reference_named_symbols()
    assert len(set(ref)) == 126               # every function kernel.h declares (zenu-cuda-kernel-sys/kernel/*.h)
    assert not [n for n in ref if not hasattr(lib, n)]
    assert lib.zenu_hip_status_string(2).decode().startswith("shape")


def test_oracle_library_builds_and_loads():
    import zenu_oracle as zo
    assert zo.lib().zo_leaf_calls() >= 0


def test_shape_errors_need_no_gpu():
    """legality is checked on the host before anything is launched"""
    import zenu_amd
    from zenu_amd import _lib
    lib = zenu_amd.lib()
    t = _lib.Tensor()
    t.ndim = 7
    assert lib.zenu_hip_unary(_lib.EXP, _lib.F32, ctypes.byref(t), ctypes.byref(t), None) == _lib.ERR_ARG
    assert lib.zenu_hip_binary(_lib.ADD, _lib.F32, None, None, None, None) == _lib.ERR_ARG
    assert lib.zenu_hip_sgd_step(_lib.F32, None, None, -1, 0.1, None) == _lib.ERR_ARG


def test_void_entry_points_leave_a_sticky_status():
    """the reference-named functions return void; the first failure behind them stays readable per
    thread until zenu_hip_last_status() clears it (host-side checks only: nothing is launched)"""
    import zenu_amd
    from zenu_amd import _lib
    lib = zenu_amd.lib()
    f = ctypes.POINTER(ctypes.c_float)
    lib.array_exp_float.argtypes = [f, ctypes.c_int, ctypes.c_int, f, ctypes.c_int]
    lib.array_exp_float.restype = None
    lib.array_array_add_float.argtypes = [f, ctypes.c_int, f, ctypes.c_int, f, ctypes.c_int, ctypes.c_int]
    lib.array_array_add_float.restype = None
    assert lib.zenu_hip_last_status() == _lib.OK
    lib.array_exp_float(None, -5, 1, None, 1)                 # a negative element count
    lib.array_array_add_float(None, 1, None, 1, None, 1, -1)  # a second failure: the first one is kept
    assert lib.zenu_hip_last_status() == _lib.ERR_ARG
    assert lib.zenu_hip_last_status() == _lib.OK              # read once, then clear
