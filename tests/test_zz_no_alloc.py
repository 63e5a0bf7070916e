"""dopt_hip_bias_bwd_noalloc: the bias gradient for callers that cannot allocate device memory.  Its partial
sums live in an array built into the library instead of the grown-on-demand workspace; the result
must equal dopt_hip_bias_bwd's bit for bit (same kernels, same fixed summation order) and the float64
oracle within the reduction tolerance, call after call, also when a smaller problem follows a larger
one in the same array."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from dopt_amd import capi, ops
from util import assert_close

pytestmark = pytest.mark.gpu


def _both(lib, dy):
    n, c = dy.shape[:2]
    inner = int(np.prod(dy.shape[2:]))
    tdy = ops.tensor(dy)
    want, got = ops.Tensor((c,)), ops.Tensor((c,))
    got.set(np.full(c, np.nan, np.float32))          # every element must be written
    capi.check(lib.dopt_hip_bias_bwd(n, c, inner, tdy.ptr, want.ptr))
    capi.check(lib.dopt_hip_bias_bwd_noalloc(n, c, inner, tdy.ptr, got.ptr))
    return got.numpy(), want.numpy()


def test_bias_gradient_without_allocation_matches_the_allocating_entry_point():
    lib = capi.load()
    capi.check(lib.dopt_hip_init(0))
    r = np.random.default_rng(7)
    live0, cached0, allocs0 = C.c_size_t(), C.c_size_t(), C.c_size_t()
    # two calls in a row on the two-stage path (inner >= 256), the second on a smaller input that
    # uses fewer partial sums than the first left behind
    big = r.standard_normal((32, 64, 32, 32)).astype(np.float32)
    small = r.standard_normal((3, 5, 16, 17)).astype(np.float32)
    for dy in (big, small):
        got, want = _both(lib, dy)
        assert np.array_equal(got, want)
        ref = O.add_bias_grad(dy)
        assert_close(got, ref, "bias gradient", scale=np.sqrt(dy.size / dy.shape[1]))
    # the one-launch path (small inner) and the empty sum
    flat = r.standard_normal((128, 10, 1, 1)).astype(np.float32)
    got, want = _both(lib, flat)
    assert np.array_equal(got, want)
    out = ops.tensor(np.full(6, 5.0, np.float32))
    capi.check(lib.dopt_hip_bias_bwd_noalloc(0, 6, 300, None, out.ptr))
    assert np.all(out.numpy() == 0)
    # nothing is taken from the pool or the driver by the call itself
    tdy, db = ops.tensor(big), ops.Tensor((64,))
    capi.check(lib.dopt_hip_pool_stats(C.byref(live0), C.byref(cached0), C.byref(allocs0)))
    capi.check(lib.dopt_hip_bias_bwd_noalloc(32, 64, 1024, tdy.ptr, db.ptr))
    live1, cached1, allocs1 = C.c_size_t(), C.c_size_t(), C.c_size_t()
    capi.check(lib.dopt_hip_pool_stats(C.byref(live1), C.byref(cached1), C.byref(allocs1)))
    assert (live0.value, cached0.value, allocs0.value) == (live1.value, cached1.value, allocs1.value)


def test_bias_gradient_without_allocation_refuses_what_its_scratch_cannot_hold():
    lib = capi.load()
    capi.check(lib.dopt_hip_init(0))
    c = 70000                                   # one slice per channel: 70000 partial sums > 65536
    dy = ops.Tensor((1, c, 256))
    db = ops.tensor(np.full(c, 2.0, np.float32))
    rc = lib.dopt_hip_bias_bwd_noalloc(1, c, 256, dy.ptr, db.ptr)
    assert rc == 1 and b"exceed the built-in scratch" in lib.dopt_hip_last_error()
    assert np.all(db.numpy() == 2.0)            # nothing was launched
    capi.check(lib.dopt_hip_bias_bwd(1, c, 256, dy.ptr, db.ptr))   # the allocating entry point takes it
    assert np.all(db.numpy() == 0.0)
