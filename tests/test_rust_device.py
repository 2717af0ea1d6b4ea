"""bindings/hip_device.rs against the reference's device traits, as text.

The image has no Rust toolchain, so the `Hip` device cannot be compiled here.  What can be checked
without one: (i) every trait that `Device` requires (zenu-matrix/src/device/mod.rs:71-109), apart
from the BLAS / cuDNN-class ones that are outside this library, has an `impl ... for Hip` in the
file, with every method the trait declares without a default body, under the same name and with the
same number of parameters; (ii) every foreign function the file calls is declared in
bindings/zenu_hip_sys.rs (which tests/test_rust_bindings.py ties to include/zenu_hip.h) and is called
with the declared number of arguments.  Needs /root/reference (the build container); skipped where
it is absent.
"""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference/zenu-matrix/src"
DEVICE_RS = os.path.join(ROOT, "bindings", "hip_device.rs")
SYS_RS = os.path.join(ROOT, "bindings", "zenu_hip_sys.rs")

pytestmark = pytest.mark.skipif(not os.path.isdir(REF), reason="the reference tree is not on this machine")

# supertraits of `Device` that are not this library's: marker traits, BLAS, and the cuDNN-class nn traits
OUTSIDE = {"Sized", "Send", "Sync", "Gemm", "BatchNormalization", "ConvFwd", "ConvBkwdData", "ConvBkwdFilter",
           "Pool2dImpl", "Dropout"}


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def _block(text, open_idx):
    """text of the brace block whose '{' is at open_idx (without the outer braces)"""
    depth = 0
    for i in range(open_idx, len(text)):
        if text[i] == "{":
            depth += 1
        elif text[i] == "}":
            depth -= 1
            if depth == 0:
                return text[open_idx + 1:i]
    raise AssertionError("unbalanced braces")


def _split_args(s):
    """top-level comma split of an argument / parameter list"""
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([{<":
            depth += 1
        elif ch in ")]}>":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur)
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur)
    return [a.strip() for a in out if a.strip()]


def _methods(trait_body, required_only):
    """name -> number of parameters for the fns declared at the top level of a trait / impl body"""
    out = {}
    for m in re.finditer(r"\bfn\s+(\w+)\s*(<[^>]*>)?\s*\(", trait_body):
        # parameters: up to the matching ')'
        start = m.end() - 1
        depth = 0
        for i in range(start, len(trait_body)):
            if trait_body[i] == "(":
                depth += 1
            elif trait_body[i] == ")":
                depth -= 1
                if depth == 0:
                    end = i
                    break
        params = _split_args(trait_body[start + 1:end])
        rest = trait_body[end + 1:]
        nxt = re.search(r"[;{]", rest)
        has_body = nxt is not None and nxt.group() == "{"
        if required_only and has_body:
            continue
        out[m.group(1)] = len(params)
    return out


def _top_level_fns(body, required_only):
    """like _methods, but ignores fns nested inside other fns' bodies"""
    flat, depth = "", 0
    for ch in body:
        if ch == "{":
            depth += 1
            if depth == 1:
                flat += "{"
            continue
        if ch == "}":
            depth -= 1
            if depth == 0:
                flat += "}"
            continue
        if depth == 0:
            flat += ch
    return _methods(flat, required_only)


def _traits_in(path):
    """trait name -> {method: n_params} for `pub trait X` blocks of a file, macro-generated ones included"""
    text = _strip_comments(open(path).read())
    traits = {}
    for m in re.finditer(r"pub trait (\$?\w+)[^{;]*\{", text):
        body = _block(text, m.end() - 1)
        name = m.group(1)
        if not name.startswith("$"):
            traits[name] = _top_level_fns(body, required_only=True)
            continue
        # a trait inside macro_rules!: one instance per invocation, the first macro argument is its name
        mac = re.findall(r"macro_rules!\s*(\w+)", text[:m.start()])[-1]
        for inv in re.finditer(mac + r"!\s*\(\s*(\w+)", text):
            traits[inv.group(1)] = _top_level_fns(body, required_only=True)
    return traits


def _reference_traits():
    dev = _strip_comments(open(os.path.join(REF, "device", "mod.rs")).read())
    m = re.search(r"pub trait Device\s*:(.*?)\{", dev, flags=re.S)
    supers = [t.strip() for t in m.group(1).split("+")]
    supers = [t for t in supers if t and not t.startswith("'")]
    wanted = [t for t in supers if t not in OUTSIDE]
    found = {}
    files = [os.path.join(REF, "device", "mod.rs"), os.path.join(REF, "nn", "conv", "interface.rs")]
    opdir = os.path.join(REF, "operation")
    files += [os.path.join(opdir, f) for f in sorted(os.listdir(opdir)) if f.endswith(".rs")]
    for f in files:
        for name, methods in _traits_in(f).items():
            found.setdefault(name, methods)
    return wanted, found


def _hip_impls():
    """trait name -> {method: n_params} implemented `for Hip` in bindings/hip_device.rs"""
    text = _strip_comments(open(DEVICE_RS).read())
    impls = {}
    for m in re.finditer(r"impl\s+(\$?\w+)\s+for\s+Hip\s*\{", text):
        body = _block(text, m.end() - 1)
        name = m.group(1)
        if not name.startswith("$"):
            impls[name] = _top_level_fns(body, required_only=False)
            continue
        mac = re.findall(r"macro_rules!\s*(\w+)", text[:m.start()])[-1]
        for inv in re.finditer(mac + r"!\s*\(\s*(\w+)", text):
            impls[inv.group(1)] = _top_level_fns(body, required_only=False)
    return impls


def test_every_required_trait_method_is_implemented_for_hip():
    wanted, ref = _reference_traits()
    assert "DeviceBase" in wanted and "AddOps" in wanted and "MaxIdx" in wanted and len(wanted) >= 24, wanted
    impls = _hip_impls()
    missing = []
    for t in wanted:
        assert t in ref, f"trait {t} not found in the reference sources"
        assert ref[t], f"no required methods parsed for {t}"
        if t not in impls:
            missing.append(f"impl {t} for Hip")
            continue
        for name, n in ref[t].items():
            if name not in impls[t]:
                missing.append(f"{t}::{name}")
            elif impls[t][name] != n:
                missing.append(f"{t}::{name} takes {impls[t][name]} parameters, the trait declares {n}")
    assert not missing, missing
    # nothing implemented that the trait does not have (a misspelt method would not compile)
    for t in wanted:
        all_methods = set(_all_methods_of(t))
        extra = set(impls[t]) - all_methods
        assert not extra, (t, extra)


def _all_methods_of(trait):
    """every method of a reference trait, defaulted ones included"""
    files = [os.path.join(REF, "device", "mod.rs"), os.path.join(REF, "nn", "conv", "interface.rs")]
    opdir = os.path.join(REF, "operation")
    files += [os.path.join(opdir, f) for f in sorted(os.listdir(opdir)) if f.endswith(".rs")]
    for f in files:
        text = _strip_comments(open(f).read())
        for m in re.finditer(r"pub trait (\$?\w+)[^{;]*\{", text):
            body = _block(text, m.end() - 1)
            names = [m.group(1)]
            if names[0].startswith("$"):
                mac = re.findall(r"macro_rules!\s*(\w+)", text[:m.start()])[-1]
                names = [i.group(1) for i in re.finditer(mac + r"!\s*\(\s*(\w+)", text)]
            if trait in names:
                return list(_top_level_fns(body, required_only=False))
    raise AssertionError(trait)


def test_device_marker_and_trait_list():
    text = open(DEVICE_RS).read()
    assert re.search(r"pub struct Hip;", text)
    assert re.search(r"impl Device for Hip \{\}", text)
    assert ".." not in re.sub(r"0\.\.\w+|\(0\.\.", "", _strip_comments(text)), "an elided body (`..`) is left in the file"
    assert "todo!" not in text and "unimplemented!()" not in text


def test_foreign_calls_are_declared_with_the_same_arity():
    sys_text = _strip_comments(open(SYS_RS).read())
    declared = {}
    for m in re.finditer(r"pub fn (\w+)\s*\(([^)]*)\)", sys_text):
        declared[m.group(1)] = len(_split_args(m.group(2)))
    assert len(declared) > 150
    text = _strip_comments(open(DEVICE_RS).read())
    calls = re.finditer(r"\b(zenu_hip_\w+|array_\w+_(?:float|double)|conv\w*_(?:float|double)|memory_\w+_(?:float|double))\s*\(", text)
    seen = set()
    for m in calls:
        name = m.group(1)
        assert name in declared, f"{name} is called but not declared in zenu_hip_sys.rs"
        start = m.end() - 1
        depth = 0
        for i in range(start, len(text)):
            if text[i] == "(":
                depth += 1
            elif text[i] == ")":
                depth -= 1
                if depth == 0:
                    end = i
                    break
        n = len(_split_args(text[start + 1:end]))
        assert n == declared[name], f"{name}: called with {n} arguments, declared with {declared[name]}"
        seen.add(name)
    # the file really goes through the library for everything it implements
    for must in ("zenu_hip_malloc", "zenu_hip_free", "zenu_hip_binary", "zenu_hip_unary", "zenu_hip_copy", "zenu_hip_sum_axis",
                 "zenu_hip_max_axis_idx", "zenu_hip_asum", "zenu_hip_adam_step_multi", "zenu_hip_sgd_step_multi"):
        assert must in seen, must
