"""The ctypes binding printed in INTEGRATION.md for a maintainer of the reference must match the
library: its `argtypes` lines are executed against the built .so and compared with the table the
package itself binds with, and every call it makes passes as many arguments as it declared."""
import ast
import ctypes
import os
import re

import pytest

from triteia_amd.python.capi import _ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def binding_snippet() -> str:
    path = os.path.join(ROOT, "INTEGRATION.md")
    if not os.path.exists(path):   # documentation does not travel to every machine the tests run on
        pytest.skip("INTEGRATION.md is not in this tree")
    text = open(path).read()
    blocks = re.findall(r"```python\n(.*?)```", text, flags=re.S)
    marlin = [b for b in blocks if "ctypes.CDLL" in b]
    assert len(marlin) == 1, "expected exactly one fenced binding with ctypes.CDLL in INTEGRATION.md"
    return marlin[0]


def test_argtypes_lines_match_the_library():
    src = binding_snippet()
    assert 'ctypes.CDLL("libtriteia_hip.so")' in src
    src = src.replace('ctypes.CDLL("libtriteia_hip.so")', f"ctypes.CDLL({_ffi.LIB_PATH!r})")
    ns = {}
    exec(compile(src, "INTEGRATION.md", "exec"), ns)   # binds argtypes, defines the three wrappers; calls nothing
    lib = ns["_lib"]
    bound = re.findall(r"_lib\.(triteia_hip_\w+)\.argtypes\s*=", src)
    assert {"triteia_hip_mul_2_4", "triteia_hip_bmm_2_4", "triteia_hip_bmm_2_4_tokens", "triteia_hip_sbmm_2_4"} <= set(bound)
    for name in bound:
        assert list(getattr(lib, name).argtypes) == list(_ffi.SIGNATURES[name][1]), name
    assert lib.triteia_hip_last_error.restype is ctypes.c_char_p
    for fn in ("mul_2_4", "bmm_2_4", "sbmm_2_4"):
        assert callable(ns[fn])


def test_every_call_passes_what_it_declared():
    tree = ast.parse(binding_snippet())
    calls = [n for n in ast.walk(tree) if isinstance(n, ast.Call) and isinstance(n.func, ast.Attribute)
             and isinstance(n.func.value, ast.Name) and n.func.value.id == "_lib" and n.func.attr.startswith("triteia_hip_")]
    seen = set()
    for c in calls:
        name = c.func.attr
        if name == "triteia_hip_last_error":
            continue
        seen.add(name)
        assert len(c.args) == len(_ffi.SIGNATURES[name][1]), f"{name}: {len(c.args)} arguments passed"
        assert not c.keywords
    assert seen == {"triteia_hip_mul_2_4", "triteia_hip_bmm_2_4", "triteia_hip_bmm_2_4_tokens", "triteia_hip_sbmm_2_4"}


def test_signature_table_matches_the_header_argument_counts():
    """include/triteia_hip.h is what a binding is written from: every prototype there has as many
    parameters as the ctypes table binds."""
    text = open(os.path.join(ROOT, "include", "triteia_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = re.findall(r"TRITEIA_HIP_API\s+[\w\s\*]+?\b(triteia_hip_\w+)\s*\(([^)]*)\)\s*;", text)
    assert len(protos) >= 12
    for name, params in protos:
        params = params.strip()
        n = 0 if params in ("", "void") else len(params.split(","))
        assert n == len(_ffi.SIGNATURES[name][1]), f"{name}: header has {n} parameters"
