"""Pointwise chains: one generated kernel against the same nodes run one kernel at a time (which the
pointwise tests pin against the oracle), bit for bit; and plans that fuse such chains against plans
that do not."""
import ctypes as C

import numpy as np
import pytest

from dopt_amd import capi, core, nnet, online, ops

pytestmark = pytest.mark.gpu
T = ops.tensor


def _one_by_one(inputs, nodes):
    vals = list(inputs)
    n = max(t.size for t in inputs)
    full = next(t for t in inputs if t.size == n)
    for i, t in enumerate(vals):
        if t.size != n:
            vals[i] = T(np.full(full.shape, t.numpy().ravel()[0], t.dtype))
    for op, lhs, rhs in nodes:
        vals.append(ops.pointwise(op, vals[lhs], None if rhs is None else vals[rhs]))
    return vals[-1].numpy()


CHAINS = [
    # w - lr * g with lr a one-element tensor (the SGD update of online/sgd.d:58-63)
    ([(1000,), (1,), (1000,)], [("mul", 1, 2), ("sub", 0, 3)]),
    # beta2 * v + (1 - beta2) * g * g                       (online/adam.d:56)
    ([(4099,), (4099,), (1,), (1,)], [("mul", 2, 0), ("mul", 3, 1), ("mul", 5, 1), ("add", 4, 6)]),
    # w - eta * (m / (sqrt(v) + eps))                        (online/adam.d:58-60)
    ([(513,), (513,), (513,), (1,), (1,)], [("sqrt", 2, None), ("add", 5, 4), ("div", 1, 6), ("mul", 3, 7), ("sub", 0, 8)]),
    # a diamond: the same node read twice, comparisons and max in the mix
    ([(33, 65), (33, 65)], [("add", 0, 1), ("mul", 2, 2), ("exp", 0, None), ("max", 3, 4), ("gt", 5, 1), ("mul", 6, 5),
                            ("tanh", 7, None)]),
    ([(7,)], [("neg", 0, None), ("abs", 1, None)]),
    ([(1 << 20,), (1 << 20,), (1,)], [("div", 0, 2), ("log", 3, None), ("atan2", 4, 1), ("min", 5, 0)]),
]


@pytest.mark.parametrize("shapes,nodes", CHAINS)
def test_chain_equals_the_nodes_run_one_by_one(shapes, nodes):
    r = np.random.default_rng(len(nodes))
    inputs = [T((np.abs(r.standard_normal(s)) + 0.5).astype(np.float32)) for s in shapes]
    got = ops.pointwise_chain(inputs, nodes).numpy()
    want = _one_by_one(inputs, nodes)
    assert np.array_equal(got, want, equal_nan=True)


def test_chain_unaligned_operands_and_int32():
    r = np.random.default_rng(0)
    base = T(r.standard_normal(1003).astype(np.float32))
    a, b = base.view(1, [1001]), base.view(2, [1001])          # 4- and 8-byte offsets: the scalar kernel
    nodes = [("mul", 0, 1), ("add", 2, 0)]
    assert np.array_equal(ops.pointwise_chain([a, b], nodes).numpy(), _one_by_one([a, b], nodes))
    ia, ib = T(r.integers(-50, 50, 300).astype(np.int32)), T(r.integers(0, 5, 300).astype(np.int32))
    nodes = [("pow", 0, 1), ("mul", 2, 0), ("sub", 3, 1)]
    assert np.array_equal(ops.pointwise_chain([ia, ib], nodes).numpy(), _one_by_one([ia, ib], nodes))


@pytest.mark.parametrize("m,n", [(7, 12), (5, 10), (128, 512), (1, 8), (9, 1), (33, 20)])
def test_chain_row_and_column_operands_and_relu_nodes(m, n):
    """relu(x + ones[m,1] . b[1,n]) and reluGrad(dy * a[m,1] . ones[1,n], x): the outer products are read as
    a per-row and a per-column element; n % 4 != 0 takes the one-element-at-a-time kernel."""
    r = np.random.default_rng(m * 100 + n)
    x = r.standard_normal((m, n)).astype(np.float32)
    dy = r.standard_normal((m, n)).astype(np.float32)
    col = r.standard_normal((m, 1)).astype(np.float32)
    row = r.standard_normal((1, n)).astype(np.float32)
    # inputs: x (tensor), col (per row), row (per column); t0 = col*row, t1 = x + t0, t2 = relu(t1)
    got = ops.pointwise_chain([T(x), T(col), T(row)], [("mul", 1, 2), ("add", 0, 3), ("relu", 4, None)],
                              kinds=[0, 2, 3], inner=n).numpy()
    outer = ops.matmul(T(col), T(row))
    want = ops.relu(ops.pointwise("add", T(x), outer)).numpy()
    assert np.array_equal(got, want)
    got = ops.pointwise_chain([T(dy), T(x), T(col), T(row)], [("mul", 2, 3), ("mul", 0, 4), ("reluGrad", 5, 1)],
                              kinds=[0, 0, 2, 3], inner=n).numpy()
    want = ops.relu_grad(ops.pointwise("mul", T(dy), outer), T(x)).numpy()
    assert np.array_equal(got, want)


def test_chain_rejects_forward_references_and_unknown_ops():
    a = T(np.ones(8, np.float32))
    with pytest.raises(capi.HipError):
        ops.pointwise_chain([a], [("add", 0, 2), ("neg", 0, None)])
    with pytest.raises(capi.HipError):
        ops.pointwise_chain([a], [("frobnicate", 0, 0)])
    assert capi.load().dopt_hip_pointwise_arity(b"atan2") == 2
    assert capi.load().dopt_hip_pointwise_arity(b"sqrt") == 1
    assert capi.load().dopt_hip_pointwise_arity(b"matmul") == 0


def _mlp(seed):
    init = nnet.Init(seed)
    x, y = core.float32([32, 20]), core.float32([32, 5])
    top = nnet.softmax(nnet.dense(nnet.relu(nnet.dense(nnet.dataSource(x), 16, init, weight_decay=1e-3)), 5, init))
    net = nnet.DAGNetwork([x], [top])
    return x, y, net, nnet.crossEntropy(top.trainOutput, y) + net.paramLoss


@pytest.mark.parametrize("maker", [online.sgd, online.adam, online.amsgrad])
def test_op_graph_optimizers_fuse_their_update_rules_without_changing_a_bit(maker):
    r = np.random.default_rng(1)
    xs = r.standard_normal((32, 20)).astype(np.float32)
    ys = np.eye(5, dtype=np.float32)[r.integers(0, 5, 32)]
    runs, kernels = [], []
    for flags in (0, core.PLAN_VIEWS | core.PLAN_FUSE):
        x, y, net, loss = _mlp(3)
        up = maker([loss], net.params, net.paramProj, flags=flags)
        losses = [up({x: xs, y: ys})[0] for _ in range(4)]
        runs.append((losses, [p.value for p in net.params]))
        kernels.append(up.plan.stats()["kernels"])
    assert kernels[1] < kernels[0] * 0.7
    for a, b in zip(runs[0][0], runs[1][0]):
        assert a == b
    for a, b in zip(runs[0][1], runs[1][1]):
        assert np.array_equal(a, b)


def test_chain_keeps_values_that_something_else_reads():
    a = core.float32([64], np.arange(64, dtype=np.float32))
    b = core.float32([64], np.ones(64, np.float32))
    s = a + b                      # read by the chain AND returned
    t = core.exp(s * 0.5) - b
    u = core.sum(s)                # a reduction reads s too
    want = core.compile([t, s, u]).execute()
    got = core.compile([t, s, u], core.PLAN_VIEWS | core.PLAN_FUSE).execute()
    for g, w in zip(got, want):
        assert np.array_equal(g, w)


def test_scalar_arithmetic_joins_the_chain_it_is_broadcast_into():
    """`weightDecay * sum(...)` differentiated gives (one-element value) x (one-element value), broadcast over the filter
    by the product with a ones vector (core/ops/basic.d:370-381): the one-element product has no kernel of its own, the
    chain over the filter computes it; the same through a `repeat`.  Values as in the plan without rewrites."""
    r = np.random.default_rng(5)
    n = 6000                                     # above the tiny-run limit
    w = core.float32([n], r.standard_normal(n).astype(np.float32))
    g = core.float32([n], r.standard_normal(n).astype(np.float32))
    u = core.float32([1], np.float32([0.37]))
    s = core.sum(g)                              # a reduction: rank 0, not part of any chain
    t = (s * 0.5) * 1.25                         # two one-element nodes, read only through the broadcast
    out = w * t + g                              # rank 0 against rank 1: repeat(t, n) = ones[n,1] x t[1,1]
    v = core.exp(u * 0.3)                        # one-element nodes again
    out2 = core.repeat(v, [n]) * w - g           # ... broadcast by a repeat
    outs = [out, out2]
    plan = core.compile(outs, core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_TIMING)
    got = plan.execute()
    prof = plan.profile()
    assert "mul" not in prof and "exp" not in prof, prof
    want = core.compile(outs).execute()
    for a, b in zip(got, want):
        assert np.array_equal(a, b)


def _random_graph(r, n_leaves=4, n_ops=18, size=96):
    """A random DAG over [size]-vectors and [8, size/8] matrices: pointwise nodes, scalar broadcasts,
    reshapes, contiguous slices padded back, reductions as side consumers, a few outputs in the middle."""
    shape2 = [8, size // 8]
    pool = [core.float32([size], (np.abs(r.standard_normal(size)) + 0.5).astype(np.float32)) for _ in range(n_leaves)]
    scalars = [core.float32([], [float(r.uniform(0.5, 1.5))]) for _ in range(2)]
    outputs = []
    for _ in range(n_ops):
        kind = r.integers(0, 10)
        a = pool[r.integers(0, len(pool))]
        b = pool[r.integers(0, len(pool))]
        if kind <= 3:
            node = [core.add, core.sub, core.mul, core.max][kind](a, b)
        elif kind == 4:
            node = core.abs(a) if r.integers(0, 2) else core.sqrt(core.abs(a))
        elif kind == 5:
            node = a * scalars[r.integers(0, 2)]                    # repeat(scalar) + reshape + mul
        elif kind == 6:
            node = core.reshape(core.reshape(a, shape2) * core.reshape(b, shape2), [size])
        elif kind == 7:
            half = size // 2
            lo = core.slice(a, [0], [half])                         # a view under PLAN_VIEWS
            node = core.pad(lo * lo, [0], [size - half])
        elif kind == 8:
            node = a + core.sum(b) * 0.01                           # a reduction reads b, its result is broadcast
        elif kind == 9 and r.integers(0, 2):
            # a dense layer's bias add and activation on the [8, size/8] view, and the activation's gradient
            bias = core.float32([shape2[1]], r.standard_normal(shape2[1]).astype(np.float32))
            pre = core.reshape(a, shape2) + core.repeat(bias, shape2[0])
            act = core.relu(pre)
            node = core.reshape(core.reluGrad(core.reshape(b, shape2), act) + act, [size])
        else:
            node = core.min(core.exp(a * 0.1), b)
        pool.append(node)
        if r.integers(0, 4) == 0:
            outputs.append(node)                                    # exposed in the middle of a would-be chain
    outputs.append(pool[-1])
    outputs.append(core.sum(pool[-2]))
    return outputs


@pytest.mark.parametrize("seed", range(20))
def test_random_graphs_give_the_same_values_with_every_rewrite(seed):
    outs = _random_graph(np.random.default_rng(100 + seed))
    want = core.compile(outs).execute()
    for flags in (core.PLAN_VIEWS, core.PLAN_VIEWS | core.PLAN_FUSE, core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_GRAPH,
                  core.PLAN_OVERLAP_LIGHT, core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_OVERLAP_LIGHT,
                  core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_OVERLAP):
        plan = core.compile(outs, flags)
        bufs = [ops.Tensor(o.shape) for o in outs]
        for _ in range(3):                                           # direct, recorded, replayed
            plan.execute(None, bufs)
            for got, w in zip(bufs, want):
                assert np.array_equal(got.numpy(), w, equal_nan=True), flags
