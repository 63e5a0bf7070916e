"""Operator-norm projections (nnet/lipschitz.d) through compiled plans.

The p=1 / p=inf norms have closed forms (numpy).  The p=2 norms are power iterations from a random
start: the plan is asked for the start vector as a second output, the iteration is redone in
float64 (matrices: numpy; convolutions: scipy.signal, an independent implementation of true
convolution and of its adjoint), and the estimate is also checked against what the mathematics
fixes - it never exceeds the largest singular value, and equals it for a rank-1 matrix.
"""
import math

import numpy as np
import pytest
import scipy.signal

from dopt_amd import core, lipschitz, nnet, online

pytestmark = pytest.mark.gpu


def _uniform_node(op):
    found = [o for o in core.topological_sort([op]) if o.opType == "uniform"]
    assert len(found) == 1
    return found[0]


def test_matrix_norm_p1_and_pinf_closed_forms():
    w = np.random.default_rng(0).standard_normal((37, 53)).astype(np.float32)
    p = core.float32(w.shape, w)
    n1, ninf = core.evaluate([lipschitz.matrixNorm(p, 1.0), lipschitz.matrixNorm(p, math.inf)])
    # the stored matrix is the transpose of the map, so p=1 is the largest absolute ROW sum
    np.testing.assert_allclose(n1, np.abs(w).sum(1).max(), rtol=1e-5)
    np.testing.assert_allclose(ninf, np.abs(w).sum(0).max(), rtol=1e-5)
    with pytest.raises(ValueError):
        lipschitz.matrixNorm(p, 3.0)
    with pytest.raises(ValueError):
        lipschitz.matrixNorm(core.float32([2, 3, 4]), 2.0)


@pytest.mark.parametrize("shape", [(10, 784), (64, 64), (512, 100)])
def test_matrix_norm_p2_power_iteration(shape):
    w = np.random.default_rng(1).standard_normal(shape).astype(np.float32)
    p = core.float32(shape, w)
    norm = lipschitz.matrixNorm(p, 2.0)
    got, u = core.evaluate([norm, _uniform_node(norm)])
    x = 2.0 * u.astype(np.float64) - 1.0
    w64 = w.astype(np.float64)
    for _ in range(2):
        x = w64 @ w64.T @ x
    v = x / np.linalg.norm(x)
    np.testing.assert_allclose(got, np.linalg.norm(w64.T @ v), rtol=1e-4)
    assert got <= np.linalg.svd(w64, compute_uv=False)[0] * (1 + 1e-5)


def test_matrix_norm_p2_exact_on_rank_one():
    r = np.random.default_rng(2)
    a, b = r.standard_normal((40, 1)) + 3.0, r.standard_normal((1, 30))   # a has no sign changes: never orthogonal to the start
    w = (np.abs(a) @ b).astype(np.float32)
    got, = core.evaluate([lipschitz.matrixNorm(core.float32(w.shape, w), 2.0)])
    np.testing.assert_allclose(got, np.linalg.norm(np.abs(a)) * np.linalg.norm(b), rtol=1e-4)


def _conv(x, k):      # true convolution, zero padding 1, one channel
    return scipy.signal.convolve2d(x, k, mode="same")


def _conv_adjoint(y, k):
    return scipy.signal.correlate2d(y, k, mode="same")


def test_conv_params_norm_reference_unittest_case():
    """nnet/lipschitz.d:148-157: the 3x3 filter 1..9 on a 200x200 image.  The reference prints the
    value without asserting one; for a non-negative filter the operator norm tends to the filter sum
    (45) as the image grows, and power iteration approaches it from below."""
    k = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
    norm = lipschitz.convParamsNorm(core.float32(k.shape, k), [200, 200], [1, 1], [1, 1], 2.0)
    got, u = core.evaluate([norm, _uniform_node(norm)])
    x = 2.0 * u.astype(np.float64)[0, 0] - 1.0
    k64 = k[0, 0].astype(np.float64)
    for _ in range(2):
        x = _conv_adjoint(_conv(x, k64), k64)
    v = x / np.linalg.norm(x)
    np.testing.assert_allclose(got, np.linalg.norm(_conv(v, k64)), rtol=1e-4)
    assert 30.0 < got <= 45.0 * (1 + 1e-5)


def test_conv_params_norm_multichannel_below_dense_operator_norm():
    r = np.random.default_rng(3)
    k = r.standard_normal((4, 3, 3, 3)).astype(np.float32)
    norm = lipschitz.convParamsNorm(core.float32(k.shape, k), [6, 6], [1, 1], [1, 1], 2.0, n=8)
    got, = core.evaluate([norm])
    # the convolution as an explicit [4*36, 3*36] matrix, column by column from unit images
    cols = []
    for c in range(3):
        for i in range(36):
            e = np.zeros((3, 6, 6))
            e[c].flat[i] = 1.0
            cols.append(np.stack([sum(_conv(e[ci], k[o, ci].astype(np.float64)) for ci in range(3)) for o in range(4)]).ravel())
    sigma = np.linalg.svd(np.array(cols).T, compute_uv=False)[0]
    assert 0.8 * sigma < got <= sigma * (1 + 1e-4)
    # p = 1 / inf fall back to the flattened matrix
    n1, = core.evaluate([lipschitz.convParamsNorm(core.float32(k.shape, k), [6, 6], [1, 1], [1, 1], 1.0)])
    np.testing.assert_allclose(n1, np.abs(k.reshape(4, -1)).sum(1).max(), rtol=1e-5)


def test_max_norm_projection():
    w = np.random.default_rng(4).standard_normal((8, 8)).astype(np.float32)
    p = core.float32(w.shape, w)
    n1 = float(np.abs(w).sum(1).max())
    shrunk, = core.evaluate([lipschitz.projMatrix(core.float32([], [n1 / 2]), 1.0)(p)])
    np.testing.assert_allclose(np.abs(shrunk).sum(1).max(), n1 / 2, rtol=1e-5)
    same, = core.evaluate([lipschitz.projMatrix(core.float32([], [n1 * 2]), 1.0)(p)])
    assert np.array_equal(same, w)


def _constrained_net(seed):
    init = nnet.Init(seed)
    x = core.float32([16, 20])
    y = core.float32([16, 5])
    bound = core.float32([], [0.5])
    h = nnet.dense(nnet.dataSource(x), 12, init, weight_proj=lipschitz.projMatrix(bound, math.inf))
    o = nnet.dense(nnet.relu(h), 5, init, weight_proj=lipschitz.projMatrix(bound, 1.0))
    net = nnet.DAGNetwork([x], [o])
    loss = nnet.squaredError(o.trainOutput, y)
    return x, y, net, loss


def test_fused_updater_applies_value_dependent_projections_like_the_graph_optimizer():
    r = np.random.default_rng(5)
    xs, ys = r.standard_normal((16, 20)).astype(np.float32), r.standard_normal((16, 5)).astype(np.float32)
    results = []
    for maker in (online.sgd, online.fused_sgd):
        x, y, net, loss = _constrained_net(7)
        up = maker([loss], net.params, net.paramProj)
        for _ in range(3):
            up({x: xs, y: ys})
        results.append([p.value for p in net.params])
    for a, b in zip(*results):
        np.testing.assert_allclose(a, b, rtol=1e-5, atol=1e-6)
    w0, w1 = results[1][0], results[1][2]
    assert np.abs(w0).sum(0).max() <= 0.5 * (1 + 1e-5)
    assert np.abs(w1).sum(1).max() <= 0.5 * (1 + 1e-5)


def test_fused_updater_rejects_projections_that_read_the_batch():
    init = nnet.Init(0)
    x = core.float32([4, 6])
    o = nnet.dense(nnet.dataSource(x), 3, init, maxgain=2.0)
    net = nnet.DAGNetwork([x], [o])
    loss = core.sum(o.trainOutput * o.trainOutput)
    with pytest.raises(NotImplementedError):
        online.fused_sgd([loss], net.params, net.paramProj)
    up = online.sgd([loss], net.params, net.paramProj)      # the op-graph optimizer takes it
    w_before = net.params[0].value
    up({x: np.random.default_rng(1).standard_normal((4, 6)).astype(np.float32)})
    assert not np.array_equal(net.params[0].value, w_before)


def test_spectral_decay_and_batchnorm_lipschitz_options_train():
    init = nnet.Init(3)
    x = core.float32([8, 3, 8, 8])
    y = core.float32([8, 4])
    c = nnet.conv2D(nnet.dataSource(x), 6, (3, 3), init, padding=(1, 1), spectral_decay=0.01)
    b = nnet.batchNorm(c, lipschitz=1.5)
    d = nnet.dense(nnet.relu(b), 4, init, spectral_decay=0.01)
    net = nnet.DAGNetwork([x], [d])
    loss = nnet.squaredError(d.trainOutput, y) + net.paramLoss
    up = online.sgd([loss], net.params, net.paramProj)
    r = np.random.default_rng(0)
    xs, ys = r.standard_normal((8, 3, 8, 8)).astype(np.float32), r.standard_normal((8, 4)).astype(np.float32)
    first = up({x: xs, y: ys})[0]
    for _ in range(20):
        last = up({x: xs, y: ys})[0]
    assert np.isfinite(last) and last < first
    gamma, var = net.params[2].value.ravel(), net.params[5].value
    assert np.abs(gamma / np.sqrt(var + 1e-6)).max() <= 1.5 * (1 + 1e-4)
