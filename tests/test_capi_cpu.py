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


def test_convolutions_refuse_tensors_their_32_bit_offsets_cannot_reach():
    """The convolution kernels address their operands with 32-bit byte offsets (buffer resources whose range
    check supplies the zero padding): a descriptor with a tensor of 2 GiB or more is refused on the host,
    before the device is touched, instead of reading zeros past the range."""
    import ctypes as C
    from dopt_amd import capi
    lib = capi.load()
    d = capi.ConvDesc(N=1 << 20, C=64, H=32, W=32, K=64, R=3, S=3, padH=1, padW=1, strideH=1, strideW=1)
    dummy = C.c_void_p(256)     # never dereferenced: the descriptor is checked first
    for call in (lambda: lib.dopt_hip_conv_fwd(C.byref(d), dummy, dummy, dummy),
                 lambda: lib.dopt_hip_conv_fwd_bias(C.byref(d), dummy, dummy, dummy, dummy),
                 lambda: lib.dopt_hip_conv_bwd_data(C.byref(d), dummy, dummy, dummy),
                 lambda: lib.dopt_hip_conv_bwd_filter(C.byref(d), dummy, dummy, dummy),
                 lambda: lib.dopt_hip_conv_fwd_bias_packed(C.byref(d), dummy, dummy, dummy, dummy),
                 lambda: lib.dopt_hip_conv_bwd_data_packed(C.byref(d), dummy, dummy, dummy)):
        assert call() == 1
        assert b"2^29 elements or more" in lib.dopt_hip_last_error()
    # a filter that large is refused as well
    d = capi.ConvDesc(N=1, C=1 << 14, H=4, W=4, K=1 << 14, R=3, S=3, padH=1, padW=1, strideH=1, strideW=1)
    assert lib.dopt_hip_conv_fwd(C.byref(d), dummy, dummy, dummy) == 1
