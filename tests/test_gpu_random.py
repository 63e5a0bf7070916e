"""`uniform` (core/ops/random.d, cuda/random.d) and dropout (nnet/layers/dropout.d).

The reference draws from cuRAND with an unpredictable seed, so its values cannot be reproduced;
what can be checked is (a) the generator itself against the published known-answer vectors of
Philox4x32-10 and an independent numpy implementation, (b) the distribution of the floats -- range
(0, 1], moments, uniformity, independence of successive calls -- and (c) the graph semantics:
fresh values on every evaluation, dropout scaling."""
import ctypes as C

import numpy as np
import pytest

from dopt_amd import capi, core, nnet, ops
from dopt_amd.core import float32

pytestmark = pytest.mark.gpu

from util import philox4x32_10


def _raw(seed, call, n):
    out = ops.Tensor((n,), np.int32)
    capi.check(capi.load().dopt_hip_philox_raw(seed, call, n, out.ptr))
    return out.numpy().view(np.uint32)


def _uniform(seed, call, n):
    out = ops.Tensor((n,))
    capi.check(capi.load().dopt_hip_uniform(seed, call, n, out.ptr))
    return out.numpy()


@pytest.mark.parametrize("seed,call,n", [(0, 0, 4), (0xA4093822299F31D0, 7, 1001), (2**64 - 1, 2**40 + 3, 70000)])
def test_device_words_are_philox(seed, call, n):
    got = _raw(seed, call, n)
    nb = (n + 3) // 4
    ctr = np.zeros((nb, 4), np.uint32)
    ctr[:, 0] = np.arange(nb) & 0xFFFFFFFF
    ctr[:, 1] = call & 0xFFFFFFFF
    ctr[:, 2] = call >> 32
    want = philox4x32_10(ctr, [seed & 0xFFFFFFFF, seed >> 32]).reshape(-1)[:n]
    assert np.array_equal(got, want)
    u = _uniform(seed, call, n)
    assert np.array_equal(u, (((want >> 8) + 1).astype(np.float64) * 2.0 ** -24).astype(np.float32))


def test_uniform_distribution():
    n = 1 << 22
    u = _uniform(12345, 0, n).astype(np.float64)
    assert u.min() > 0.0 and u.max() <= 1.0                       # (0, 1], as curandGenerateUniform
    assert abs(u.mean() - 0.5) < 5 / np.sqrt(12 * n)              # 5 sigma
    assert abs(u.var() - 1 / 12) < 5 * np.sqrt(1 / 180 / n)
    counts = np.bincount(np.minimum((u * 64).astype(np.int64), 63), minlength=64)
    chi2 = ((counts - n / 64) ** 2 / (n / 64)).sum()
    assert chi2 < 63 + 6 * np.sqrt(2 * 63)                        # chi-square, 63 degrees of freedom
    # successive elements and successive calls are uncorrelated
    assert abs(np.corrcoef(u[:-1], u[1:])[0, 1]) < 5 / np.sqrt(n)
    v = _uniform(12345, 1, n).astype(np.float64)
    assert abs(np.corrcoef(u, v)[0, 1]) < 5 / np.sqrt(n)
    assert not np.array_equal(_uniform(12346, 0, 1000), u[:1000].astype(np.float32))


def test_uniform_operation_gives_fresh_values_each_evaluation():
    a = core.uniformSample([3, 1000])
    b = core.uniformSample([3, 1000])
    plan = core.compile([a, b, a + b])
    x1, y1, s1 = plan.execute()
    x2, y2, _ = plan.execute()
    assert x1.shape == (3, 1000) and x1.dtype == np.float32
    assert 0 < x1.min() and x1.max() <= 1
    assert not np.array_equal(x1, x2) and not np.array_equal(y1, y2)     # new draws per evaluation
    assert not np.array_equal(x1, y1)                                    # two operations, two streams
    assert np.array_equal(s1, x1 + y1)                                   # one draw per evaluation, shared by readers


def test_dropout_layer():
    x = float32([64, 4096])
    X = np.random.default_rng(3).standard_normal((64, 4096)).astype(np.float32)
    layer = nnet.dropout(nnet.dataSource(x), 0.3)
    y_eval, y_train = core.evaluate([layer.output, layer.trainOutput], {x: X})
    assert np.array_equal(y_eval, X * np.float32(0.7))                   # inference: scale by 1 - p
    kept = y_train != 0
    assert np.array_equal(y_train[kept], X[kept])                        # training: mask only, no rescaling
    frac = kept.mean()
    assert abs(frac - 0.7) < 5 * np.sqrt(0.21 / X.size)
