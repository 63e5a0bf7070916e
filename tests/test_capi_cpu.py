"""No-GPU checks of the boundary: the library loads, exports every symbol the header declares,
its run-time templates compile for gfx950, and argument errors surface as the reference's
`enforce` failures would."""
import ctypes as C
import os
import re

import pytest

from dopt_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dopt_hip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = _declared("dopt_hip.h")
    assert len(names) >= 45
    for n in names:
        assert hasattr(lib, n), n
    assert set(names) == set(capi.exported_symbols())


def test_plan_header_symbols_exported():
    lib = capi.load()
    path = os.path.join(ROOT, "include", "dopt_hip_plan.h")
    if not os.path.exists(path):
        pytest.skip("plan header not present")
    for n in _declared("dopt_hip_plan.h"):
        assert hasattr(lib, n), n


@pytest.mark.parametrize("dtype", [capi.F32, capi.I32])
def test_every_rtc_template_compiles_for_gfx950(dtype):
    lib = capi.load()
    ops = ["add", "sub", "mul", "div", "lt", "lte", "gt", "gte", "eq", "neq", "max", "min", "pow", "atan2",
           "neg", "abs", "sgn", "exp", "log", "sqrt", "sin", "tanh", "sum", "maxElement", "argmin"]
    for op in ops:
        rc = lib.dopt_hip_rtc_compile_only(op.encode(), dtype, b"gfx950")
        assert rc == 0, (op, lib.dopt_hip_last_error())


def test_errors_are_reported_not_swallowed():
    lib = capi.load()
    assert lib.dopt_hip_rtc_compile_only(b"nosuchop", capi.F32, b"gfx950") == 3
    assert b"nosuchop" in lib.dopt_hip_last_error()
    assert lib.dopt_hip_rtc_compile_only(b"add", 7, b"gfx950") == 3
    assert lib.dopt_hip_last_error() == b"Element type not supported."   # cuda/math.d:237-240
    with pytest.raises(capi.HipError):
        capi.check(lib.dopt_hip_malloc(None, 16))
    # zero-byte buffers are legal and empty (cuda/package.d:144-147)
    p = C.c_void_p(1)
    assert lib.dopt_hip_malloc(C.byref(p), 0) == 0 and not p.value
    assert lib.dopt_hip_free(None) == 0
