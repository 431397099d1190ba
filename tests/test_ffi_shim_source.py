"""The jax.ffi shim is committed as source and cannot be compiled here (no jax, no XLA headers).  What can be checked
without them: the Python side parses, both sides name the same targets, every C-ABI entry point a handler calls is
declared in include/rpa_hip.h with as many arguments as the call passes, and the aliasing the Python side declares
points at the operands the handlers check."""

import ast
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _read(*parts):
    with open(os.path.join(ROOT, *parts)) as f:
        return f.read()


def _split_args(text):
    """Top-level comma split of an argument list."""
    out, depth, cur = [], 0, ""
    for ch in text:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip())
            cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


def _call_args(src, name):
    """Argument lists of every call of `name(` in C source (comments removed)."""
    src = re.sub(r"//[^\n]*", "", src)
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    found = []
    for m in re.finditer(r"\b%s\s*\(" % re.escape(name), src):
        i, depth = m.end(), 1
        while depth:
            depth += {"(": 1, ")": -1}.get(src[i], 0)
            i += 1
        found.append(_split_args(src[m.end():i - 1]))
    return found


def test_python_side_parses_and_names_the_handlers_of_the_c_side():
    py = _read("easydel_amd", "ffi_calls.py")
    tree = ast.parse(py)
    targets = next(ast.literal_eval(n.value) for n in ast.walk(tree)
                   if isinstance(n, ast.Assign) and getattr(n.targets[0], "id", "") == "TARGETS")
    cc = _read("easydel_amd", "csrc", "rpa_ffi.cc")
    handlers = re.findall(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*(\w+)\s*,\s*(\w+)", cc)
    assert sorted(targets) == sorted(h for h, _ in handlers) and len(handlers) == 7
    used = set(re.findall(r'ffi_call\(\s*"(\w+)"', py))
    assert used == set(targets), "every registered target has a wrapper"
    for _, impl in handlers:
        assert re.search(r"ffi::Error\s+%s\s*\(" % impl, cc), f"{impl} is bound but not defined"


def test_handlers_call_the_c_abi_with_the_declared_number_of_arguments():
    header = _read("include", "rpa_hip.h")
    cc = _read("easydel_amd", "csrc", "rpa_ffi.cc")
    called = set(re.findall(r"\b(rpa_[a-z0-9_]+)\s*\(", re.sub(r"//[^\n]*", "", cc))) - {"rpa_last_error"}
    assert {"rpa_ragged_paged_attention", "rpa_ragged_paged_attention_v3", "rpa_ragged_paged_attention_v3_quantised",
            "rpa_unified_attention", "rpa_page_scatter_slices", "rpa_page_scatter_ragged", "rpa_mla_ragged_paged_attention"} == called
    for name in called:
        decl = _call_args(header, name)
        assert len(decl) == 1, name
        for args in _call_args(cc, name):
            assert len(args) == len(decl[0]), f"{name}: the handler passes {len(args)} arguments, the header declares {len(decl[0])}"


def test_binding_arity_matches_the_handler_signatures():
    cc = re.sub(r"//[^\n]*", "", _read("easydel_amd", "csrc", "rpa_ffi.cc"))
    for handler, impl in re.findall(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(\s*(\w+)\s*,\s*(\w+)", cc):
        bind = cc[cc.index("XLA_FFI_DEFINE_HANDLER_SYMBOL(" + handler):]
        bind = bind[:bind.index(");") + 2].replace("RPA_ATTENTION_ATTRS", '.Attr<float>("a").Attr<int32_t>("b").Attr<float>("c")')
        n_bound = len(re.findall(r"\.(?:Ctx|Arg|Ret|Attr)<", bind))
        params = _call_args(cc, "ffi::Error " + impl)[0]
        assert n_bound == len(params), f"{handler}: {n_bound} bound items, {impl} takes {len(params)} parameters"


def test_shim_type_checks_against_a_stub_of_the_ffi_api():
    """The handler file compiles (syntax and types only) against tests/ffi_api_stub, a stand-in with the shape of the
    XLA FFI API the file uses: every handler's parameter list matches, type by type, what its binding declares.  This
    is not a build against jaxlib's header, which the image does not have."""
    import shutil
    import subprocess

    gxx = shutil.which("g++")
    hip_include = "/opt/rocm/include"
    if gxx is None or not os.path.exists(os.path.join(hip_include, "hip", "hip_runtime.h")):
        pytest.skip("needs g++ and the HIP headers")
    cmd = [gxx, "-fsyntax-only", "-std=c++17", "-D__HIP_PLATFORM_AMD__", "-I" + hip_include,
           "-I" + os.path.join(ROOT, "tests", "ffi_api_stub"), os.path.join(ROOT, "easydel_amd", "csrc", "rpa_ffi.cc")]
    done = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-3000:]
