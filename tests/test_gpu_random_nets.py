"""Randomly assembled small networks through compiled plans: every layer order the builders allow, not only the
ones the benchmark configurations use (convolution with and without bias, batch norm with and without a relu
behind it or in front of it, pools in any place, 1x1 and strided convolutions, residual sums, dense layers with
a batch norm in between).  Loss, predictions, every parameter gradient and the running statistics are compared
with the CPU evaluator, and the plans with rewrites against the plan without them: the rewrites are pattern
matches on the graph, and a pattern that fires on a neighbourhood it was not written for shows up here.
(Found this way: a transpose folded into a product whose kernel then summed in another order; the steps behind a
convolution without batch norm dropped from plans that move small steps to the second queue, and fused
convolution + bias steps moved there ahead of the step that packs their filter.)
"""
import numpy as np
import pytest

from dopt_amd import core, nnet, online, workloads
from dopt_amd.core import float32, grad
from oracle import evaluator
from util import assert_close

pytestmark = pytest.mark.gpu

REWRITES = core.PLAN_VIEWS | core.PLAN_FUSE


def _residual(a, b):
    return nnet.Layer([a, b], a.output + b.output, a.trainOutput + b.trainOutput, [])


def _as_images(layer):
    n, c = layer.output.shape
    return nnet.Layer([layer], layer.output.reshape([n, c, 1, 1]), layer.trainOutput.reshape([n, c, 1, 1]), [])


def _random_net(r, feats, widths=(8, 16, 24, 32, 64)):
    init = nnet.Init(int(r.integers(1 << 30)))
    layer = nnet.dataSource(feats)

    def size():
        return layer.output.shape[2]

    def decay():
        return float(r.choice([0.0, 0.0, 5e-4]))

    for _ in range(int(r.integers(2, 5))):
        channels = int(r.choice(widths))
        entry = layer
        shape = int(r.integers(0, 10))
        bias = bool(r.integers(0, 2))
        if shape == 0:
            conv = nnet.conv2D(layer, channels, (1, 1), init, use_bias=bias, weight_decay=decay())
        elif shape == 1 and size() >= 8:
            conv = nnet.conv2D(layer, channels, (3, 3), init, padding=(1, 1), stride=(2, 2), use_bias=bias)
        elif shape == 2 and size() >= 8:
            conv = nnet.conv2D(layer, channels, (3, 3), init, use_bias=bias)                    # no padding: the image shrinks
        elif shape == 3 and size() >= 8:
            conv = nnet.conv2D(layer, channels, (5, 5), init, padding=(2, 2), use_bias=bias, weight_decay=decay())
        else:
            conv = nnet.conv2D(layer, channels, (3, 3), init, padding=(1, 1), use_bias=bias, weight_decay=decay())
        order = int(r.integers(0, 6))
        if order == 0:
            layer = nnet.relu(nnet.batchNorm(conv))
        elif order == 1:
            layer = nnet.relu(conv)
        elif order == 2:
            layer = nnet.batchNorm(conv)
        elif order == 3:
            layer = nnet.batchNorm(nnet.relu(conv))
        elif order == 4 and entry.output.shape[2] % conv.output.shape[2] == 0:
            # a residual block: the entry reaches the sum through a 1x1 projection of the same stride
            stride = (entry.output.shape[2] // conv.output.shape[2],) * 2
            shortcut = nnet.conv2D(entry, channels, (1, 1), init, stride=stride, use_bias=False)
            layer = _residual(nnet.relu(nnet.batchNorm(conv)), shortcut)
        else:
            layer = conv
        if size() >= 4 and size() % 2 == 0 and r.integers(0, 2):
            layer = nnet.maxPool(layer, (2, 2))
            if r.integers(0, 3) == 0:
                layer = nnet.relu(layer)
    if r.integers(0, 4) == 0:
        layer = nnet.meanPool(layer)           # the Wide-ResNet head: a row sum, which `sum` turns into a GEMV
    for _ in range(int(r.integers(0, 3))):
        width = int(r.choice([12, 32, 40]))
        dense = nnet.dense(layer, width, init, use_bias=bool(r.integers(0, 2)), weight_decay=decay())
        head = int(r.integers(0, 4))
        if head == 0:
            layer = nnet.relu(nnet.batchNorm(_as_images(dense)))
        elif head == 1:
            layer = nnet.relu(dense)
        elif head == 2:
            layer = nnet.batchNorm(_as_images(dense))
        else:
            layer = dense
    return nnet.softmax(nnet.dense(layer, 10, init))


@pytest.mark.parametrize("seed", range(60))
def test_random_networks_match_the_cpu_evaluator_with_and_without_rewrites(seed):
    r = np.random.default_rng(4000 + seed)
    n = int(r.choice([4, 8]))
    size = int(r.choice([8, 16]))
    cin = int(r.choice([3, 16]))
    X = r.standard_normal((n, cin, size, size)).astype(np.float32)
    Y = workloads.one_hot(r.integers(0, 10, n))
    feats, labels = float32([n, cin, size, size]), float32([n, 10])
    preds = _random_net(r, feats)
    net = nnet.DAGNetwork([feats], [preds])
    if r.integers(0, 2):
        loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    else:
        loss = nnet.squaredError(preds.trainOutput, labels) + net.paramLoss
    stats = [net.paramProj[p](p) for p in net.params if p in net.paramProj]
    outs = [loss, preds.trainOutput, preds.output] + grad(loss, net.params) + stats
    args = {feats: X, labels: Y}
    want = evaluator.evaluate(outs, args)
    plain = core.compile(outs, 0).execute(args)
    for i, (g, w) in enumerate(zip(plain, want)):
        # A gradient is a sum over up to a few thousand products and some of its elements nearly cancel: its rounding
        # error follows the tensor's largest values, not each element's own.  This test looks for wrong wiring, whose
        # errors are of the size of the values; rounding per operation is accounted for in the operation tests.
        assert_close(g, w, "seed %d output %d (%s %s)" % (seed, i, outs[i].opType, outs[i].shape),
                     scale=10.0 * max(1.0, float(np.abs(w).max()) if np.size(w) else 1.0))
    for flags in (core.PLAN_VIEWS, REWRITES, REWRITES | core.PLAN_GRAPH, REWRITES | core.PLAN_OVERLAP_LIGHT,
                  REWRITES | core.PLAN_OVERLAP):
        plan = core.compile(outs, flags)
        for rep in range(3 if flags & core.PLAN_GRAPH else 1):     # direct, recorded, replayed
            got = plan.execute(args)
            for i, (g, p) in enumerate(zip(got, plain)):
                what = "seed %d flags %d run %d output %d (%s %s)" % (seed, flags, rep, i, outs[i].opType, outs[i].shape)
                if np.ndim(p) <= 1:
                    # bias gradients in front of a batch norm are sums whose exact value is zero, taken in the fused
                    # kernel's order; every other vector is held to the same bits as well
                    if not np.array_equal(g, p):
                        assert_close(g, p, what, scale=max(1.0, float(np.abs(p).max()) if np.size(p) else 1.0))
                else:
                    assert np.array_equal(g, p), what
        plan.cleanup()


@pytest.mark.parametrize("seed", range(48))
def test_random_wider_networks_give_the_same_values_with_the_rewrites(seed):
    """The same at sizes where the tiled convolution kernels, packed filters, one-launch backward pairs and results
    left as partial copies come into play (the small networks above mostly take the generic kernels): the plans with
    rewrites against the plan without them, whose kernels the operation tests hold against the oracle one by one."""
    r = np.random.default_rng(5000 + seed)
    n = int(r.choice([16, 32]))
    size = int(r.choice([16, 32]))
    cin = int(r.choice([3, 16, 64]))
    X = r.standard_normal((n, cin, size, size)).astype(np.float32)
    Y = workloads.one_hot(r.integers(0, 10, n))
    feats, labels = float32([n, cin, size, size]), float32([n, 10])
    preds = _random_net(r, feats, widths=(32, 64, 128))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    stats = [net.paramProj[p](p) for p in net.params if p in net.paramProj]
    outs = [loss, preds.trainOutput, preds.output] + grad(loss, net.params) + stats
    args = {feats: X, labels: Y}
    plain = core.compile(outs, 0).execute(args)
    assert all(np.isfinite(p).all() for p in plain)
    for flags in (core.PLAN_VIEWS, REWRITES, REWRITES | core.PLAN_GRAPH, REWRITES | core.PLAN_OVERLAP_LIGHT,
                  REWRITES | core.PLAN_OVERLAP):
        plan = core.compile(outs, flags)
        for rep in range(3 if flags & core.PLAN_GRAPH else 1):
            got = plan.execute(args)
            for i, (g, p) in enumerate(zip(got, plain)):
                what = "seed %d flags %d run %d output %d (%s %s)" % (seed, flags, rep, i, outs[i].opType, outs[i].shape)
                if np.ndim(p) <= 1:
                    if not np.array_equal(g, p):
                        assert_close(g, p, what, scale=max(1.0, float(np.abs(p).max()) if np.size(p) else 1.0))
                else:
                    assert np.array_equal(g, p), what
        plan.cleanup()


@pytest.mark.parametrize("seed", range(18))
def test_random_networks_fused_updaters_follow_the_op_graph_updaters(seed):
    """Two steps of SGD (plain, momentum, Nesterov), ADAM or AMSGrad on a random network: the fused update kernels
    leave the parameters and report the losses the reference's op-graph update rules do, bit for bit, with and
    without the plan rewrites."""
    rule = seed % 3
    after = []
    for fused in (False, True):
        for flags in (0, REWRITES):
            r = np.random.default_rng(6000 + seed)
            n, size, cin = int(r.choice([4, 8])), int(r.choice([8, 16])), int(r.choice([3, 16]))
            X = r.standard_normal((n, cin, size, size)).astype(np.float32)
            Y = workloads.one_hot(r.integers(0, 10, n))
            feats, labels = float32([n, cin, size, size]), float32([n, 10])
            preds = _random_net(r, feats)
            net = nnet.DAGNetwork([feats], [preds])
            loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
            if rule == 0:
                mu, nesterov = float(r.choice([0.0, 0.9])), bool(r.integers(0, 2))
                if fused:
                    up = online.fused_sgd([loss], net.params, net.paramProj, 0.05, mu, nesterov, flags=flags)
                else:
                    up = online.sgd([loss], net.params, net.paramProj, float32([], [0.05]), float32([], [mu]), nesterov, flags=flags)
            elif rule == 1:
                up = (online.fused_adam if fused else online.adam)([loss], net.params, net.paramProj, flags=flags)
            else:
                up = (online.fused_amsgrad if fused else online.amsgrad)([loss], net.params, net.paramProj, flags=flags)
            losses = [up({feats: X, labels: Y})[0] for _ in range(2)]
            after.append((fused, flags, losses, [p.value.copy() for p in net.params]))
            del up
    for flags in (0, REWRITES):
        graph, fusedrun = [a for a in after if a[1] == flags]
        assert not graph[0] and fusedrun[0]
        assert np.isfinite(graph[2]).all() and graph[2][0] != graph[2][1], graph[2]
        assert graph[2] == fusedrun[2], (seed, flags, graph[2], fusedrun[2])
        for i, (a, b) in enumerate(zip(graph[3], fusedrun[3])):
            assert np.array_equal(a, b), (seed, flags, i, a.shape)


@pytest.mark.parametrize("seed", range(150))
def test_random_networks_inference_plans_in_every_mode(seed):
    """The inference output alone: every step of such a plan leads to its one output, so the second-queue mode for small
    steps moves whole tails of the network.  The FIRST execution is compared as well as later ones: a convolution that
    ran ahead of the step packing its filter read an empty packed copy once and was right from then on."""
    r = np.random.default_rng(9000 + seed)
    n, size, cin = int(r.choice([4, 8, 16])), int(r.choice([8, 16])), int(r.choice([3, 16]))
    X = r.standard_normal((n, cin, size, size)).astype(np.float32)
    feats = float32([n, cin, size, size])
    preds = _random_net(r, feats)
    want = core.compile([preds.output], 0).execute({feats: X})[0]
    assert np.isfinite(want).all()
    for flags in (core.PLAN_VIEWS, REWRITES, REWRITES | core.PLAN_GRAPH, REWRITES | core.PLAN_OVERLAP_LIGHT,
                  REWRITES | core.PLAN_OVERLAP, core.PLAN_OVERLAP_LIGHT):
        plan = core.compile([preds.output], flags)
        for rep in range(3):
            assert np.array_equal(plan.execute({feats: X})[0], want), (seed, flags, rep)
        plan.cleanup()
