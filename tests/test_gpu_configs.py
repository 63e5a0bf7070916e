"""The benchmark configurations as parity cases: whole training steps (or the whole fused update)
run through compiled plans on the GPU and compared with the CPU oracle on the same seeded inputs.

  config 1  softmax regression as examples/mnistlogit.d writes it: whole steps against the CPU evaluator
  config 2  MLP 784-512-512-10, batch 256, one ADAM step (op-graph form and fused form)
  config 3  fused ADAM / AMSGrad over 16 777 216 parameters in 40 tensors (full size, bit-exact)
  config 4  VGG-16 + batch norm, the benchmark itself: tests/test_gpu_config4.py
  config 5  Wide-ResNet-28-10 convolution shapes (stride 2, 1x1 projections): oracle parity at a
            reduced batch, adjoint identities at batch 128, one residual block against the oracle
"""
import numpy as np
import pytest

import oracle as O
from dopt_amd import configs, core, nnet, online, ops, workloads
from oracle import evaluator
from dopt_amd.core import float32, grad
from util import assert_close

pytestmark = pytest.mark.gpu
T = ops.tensor


def _f(shape, vals):
    return float32(list(shape), np.asarray(vals, np.float32).reshape(-1))


# ------------------------------------------------------------------------------ config 1
@pytest.mark.parametrize("flags", [0, configs.REWRITES, configs.REWRITES | core.PLAN_GRAPH], ids=["plain", "rewrites", "graph"])
def test_config1_whole_steps_match_the_cpu_evaluator(flags):
    """The one configuration the reference's CPU backend can train: every output of the update plan (loss,
    predictions, new weights, new bias, new momenta) against the same graph evaluated on the CPU, one
    restated reference kernel per operation (cpu/package.d:182-280), over three consecutive steps."""
    step = configs.softmax_regression(flags=flags, host_args=(flags & core.PLAN_GRAPH) == 0)
    outs = step.updater.plan.outputs
    host_args = {k: (v if isinstance(v, np.ndarray) else v.numpy()) for k, v in step.args.items()}
    W, b = step.params
    losses = []
    for it in range(3):
        want = evaluator.evaluate(outs, host_args)          # reads the variables' current values
        got_loss, got_preds = step.updater(step.args)        # runs the step and writes the variables back
        assert_close(got_loss, want[0], "loss, step %d" % it)
        assert_close(got_preds, want[1], "predictions, step %d" % it)
        assert_close(W.value, want[2], "weights after step %d" % it)
        assert_close(b.value, want[3], "bias after step %d" % it)
        losses.append(float(got_loss))
    assert losses[0] == pytest.approx(np.log(10), rel=1e-4)   # zero weights: uniform predictions
    assert losses[2] < losses[1] < losses[0]


# ------------------------------------------------------------------------------ config 2
def _mlp_oracle(X, Y, Ws, bs):
    """Forward and backward of dense-relu-dense-relu-dense-softmax + cross entropy; GEMMs in float64."""
    acts, pre, a = [X], [], X
    for i, (W, b) in enumerate(zip(Ws, bs)):
        z = (a.astype(np.float64) @ W.astype(np.float64).T + b).astype(np.float32)   # layers/dense.d: x . W^T + b
        pre.append(z)
        a = O.relu(z) if i < 2 else O.softmax(z, f64=True)
        acts.append(a)
    p = a.astype(np.float64)
    n = X.shape[0]
    loss = -(Y * np.log(p + 1e-6)).sum() / n                                          # nnet/losses.d:23-26
    dp = (-(Y / (p + 1e-6)) / n).astype(np.float32)
    dz = O.softmax_grad(dp, a)
    gW, gb = [None] * 3, [None] * 3
    for i in (2, 1, 0):
        gW[i] = dz.astype(np.float64).T @ acts[i].astype(np.float64)
        gb[i] = dz.astype(np.float64).sum(axis=0)
        if i:
            da = (dz.astype(np.float64) @ Ws[i].astype(np.float64)).astype(np.float32)
            dz = O.relu_grad(da, pre[i - 1])
    return loss, p, gW, gb


def _mlp_problem():
    X = np.random.default_rng(0).random((256, 784)).astype(np.float32)
    Y = workloads.one_hot(np.random.default_rng(1).integers(0, 10, 256))
    feats, labels = float32([256, 784]), float32([256, 10])
    init = nnet.Init(2)
    body = nnet.dataSource(feats)
    body = nnet.relu(nnet.dense(body, 512, init))
    body = nnet.relu(nnet.dense(body, 512, init))
    preds = nnet.softmax(nnet.dense(body, 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    return X, Y, feats, labels, net, loss, preds


@pytest.mark.parametrize("fused", [False, True])
def test_config2_mlp_adam_step(fused):
    X, Y, feats, labels, net, loss, preds = _mlp_problem()
    W0 = [p.value.copy() for p in net.params]
    want_loss, want_p, gW, gb = _mlp_oracle(X, Y, W0[0::2], W0[1::2])
    make = online.fused_adam if fused else online.adam
    up = make([loss, preds.trainOutput], net.params)
    got_loss, got_p = up({feats: X, labels: Y})
    assert_close(got_loss, want_loss, "loss")
    assert_close(got_p, want_p, "predictions")
    if fused:
        m = [t.numpy() for t in up.state["m"]]
        v = [t.numpy() for t in up.state["v"]]
    else:
        m, v = [x.value for x in up.means], [x.value for x in up.vars]
    b1, b2, eta = O.adam_scalars(1e-3, 0.9, 0.999, 1.0, 1.0)
    for i, p in enumerate(net.params):
        g64 = (gW[i // 2] if i % 2 == 0 else gb[i // 2]).reshape(p.shape)
        # first step from zero moments: m' = 0.1 g and v' = 0.001 g^2 pin the gradients themselves
        # (a 784- or 512- or 256-term reduction each, hence the scaled atol)
        assert_close(m[i], 0.1 * g64, "first moment of parameter %d" % i, scale=0.1 * 16)
        assert_close(v[i], 0.001 * g64 * g64, "second moment of parameter %d" % i, rtol=3e-4, scale=1e-3)
        moved = np.abs(p.value - W0[i])
        nz = np.abs(g64) > 1e-4
        # |w' - w| = eta m'/(sqrt(v')+eps) ~= alpha wherever sqrt(v') = 0.0316 |g| is well above eps
        assert np.allclose(moved[nz], 1e-3, rtol=2e-2), i
        assert not moved[np.asarray(g64) == 0].any(), i
    if not fused:
        assert up.b1.value == np.float32(b1) and up.b2.value == np.float32(b2)


def test_config2_fused_and_op_graph_adam_agree_bit_for_bit():
    results = []
    for make in (online.adam, online.fused_adam):
        X, Y, feats, labels, net, loss, preds = _mlp_problem()
        up = make([loss], net.params)
        for _ in range(3):
            up({feats: X, labels: Y})
        results.append([p.value.copy() for p in net.params])
    for a, b in zip(*results):
        assert np.array_equal(a, b)


# ------------------------------------------------------------------------------ config 3
@pytest.mark.parametrize("rule", ["adam", "amsgrad"])
def test_config3_fused_update_16m_params_bit_exact(rule):
    st = workloads.adam16m_state(0)
    assert sum(s["w"].size for s in st) == 1 << 24 and len(st) == 40
    tw, tg, tm, tv, tvh = ([T(s[k]) for s in st] for k in ("w", "g", "m", "v", "vhat"))
    opt = ops.FusedOptimizer(tw, tg, tm, tv, tvh if rule == "amsgrad" else None)
    b1 = b2 = 1.0
    for step in range(2):
        getattr(opt, rule)(1e-3, 0.9, 0.999, 1e-8)
        b1, b2, eta = O.adam_scalars(1e-3, 0.9, 0.999, b1, b2)
        for s in st:
            if rule == "adam":
                s["w"], s["m"], s["v"] = O.adam_step(s["w"], s["g"], s["m"], s["v"], eta)
            else:
                s["w"], s["m"], s["v"], s["vhat"] = O.amsgrad_step(s["w"], s["g"], s["m"], s["v"], s["vhat"], eta)
    for i, s in enumerate(st):
        assert np.array_equal(tw[i].numpy(), s["w"]), ("w", i)
        assert np.array_equal(tm[i].numpy(), s["m"]), ("m", i)
        assert np.array_equal(tv[i].numpy(), s["v"]), ("v", i)
        assert np.array_equal(tg[i].numpy(), st[i]["g"]), ("g untouched", i)
        if rule == "amsgrad":
            assert np.array_equal(tvh[i].numpy(), s["vhat"]), ("vhat", i)


# ------------------------------------------------------------------------------ config 5
WRN_LAYERS = [  # (C, K, H, R, pad, stride) of every distinct convolution of Wide-ResNet-28-10
    (3, 16, 32, 3, 1, 1), (16, 160, 32, 3, 1, 1), (160, 160, 32, 3, 1, 1), (16, 160, 32, 1, 0, 1),
    (160, 320, 32, 3, 1, 2), (320, 320, 16, 3, 1, 1), (160, 320, 32, 1, 0, 2),
    (320, 640, 16, 3, 1, 2), (640, 640, 8, 3, 1, 1), (320, 640, 16, 1, 0, 2),
]


def _wrn_case(layer, n, seed):
    c, k, h, r, pad, st = layer
    g = np.random.default_rng(seed)
    x = g.standard_normal((n, c, h, h)).astype(np.float32)
    w = (g.standard_normal((k, c, r, r)) * np.sqrt(2.0 / (c * r * r))).astype(np.float32)
    p = (h + 2 * pad - r) // st + 1
    dy = g.standard_normal((n, k, p, p)).astype(np.float32)
    return x, w, dy, (pad, pad), (st, st)


@pytest.mark.parametrize("layer", WRN_LAYERS, ids=lambda l: "c%dk%dh%dr%ds%d" % (l[0], l[1], l[2], l[3], l[5]))
def test_config5_wrn_conv_shapes_match_the_oracle_at_reduced_batch(layer):
    # the float64 direct loops finish in seconds at batch 2; channel counts, extents, strides and
    # padding are the real ones
    x, w, dy, pad, st = _wrn_case(layer, 2, 50)
    red = layer[0] * layer[3] ** 2
    assert_close(ops.convolution(T(x), T(w), pad, st).numpy(), O.convolution(x, w, pad, st), "fwd", scale=1.0)
    assert_close(ops.conv_bwd_data(T(dy), T(w), x.shape, pad, st).numpy(),
                 O.conv_bwd_data(dy, w, x.shape, pad, st), "bwd-data", scale=np.sqrt(layer[1] * layer[3] ** 2 / red))
    assert_close(ops.conv_bwd_filter(T(dy), T(x), w.shape, pad, st).numpy(),
                 O.conv_bwd_filter(dy, x, w.shape, pad, st), "bwd-filter", scale=np.sqrt(dy[0, 0].size * 2.0))
    # the same two gradients from an upstream gradient of the size a mean loss hands down (He-scaled
    # weights already keep the forward result O(1)): stated tolerance with no rescaling
    dys = (dy * np.float32(1.0 / dy[0, 0].size)).astype(np.float32)
    assert_close(ops.conv_bwd_data(T(dys), T(w), x.shape, pad, st).numpy(),
                 O.conv_bwd_data(dys, w, x.shape, pad, st), "bwd-data, mean-loss gradient")
    assert_close(ops.conv_bwd_filter(T(dys), T(x), w.shape, pad, st).numpy(),
                 O.conv_bwd_filter(dys, x, w.shape, pad, st), "bwd-filter, mean-loss gradient")


@pytest.mark.parametrize("layer", WRN_LAYERS[4:], ids=lambda l: "c%dk%dh%dr%ds%d" % (l[0], l[1], l[2], l[3], l[5]))
def test_config5_wrn_conv_adjoint_identities_at_batch_128(layer):
    # <conv(x,w), dy> = <x, bwdData(dy,w)> = <w, bwdFilter(dy,x)>: fixes the three kernels against
    # each other at the full size, where the direct loops would take minutes
    x, w, dy, pad, st = _wrn_case(layer, 128, 51)
    y = ops.convolution(T(x), T(w), pad, st).numpy().astype(np.float64)
    dx = ops.conv_bwd_data(T(dy), T(w), x.shape, pad, st).numpy().astype(np.float64)
    dw = ops.conv_bwd_filter(T(dy), T(x), w.shape, pad, st).numpy().astype(np.float64)
    a, b, c = (y * dy).sum(), (dx * x).sum(), (dw * w).sum()
    mag = np.sqrt((y * y).sum() * (dy.astype(np.float64) ** 2).sum())
    assert abs(a - b) < 1e-5 * mag and abs(a - c) < 1e-5 * mag, (a, b, c, mag)
    # and linearity in the filter at full size: conv(x, 2w) = 2 conv(x, w) exactly (power of two)
    y2 = ops.convolution(T(x), T(w * np.float32(2)), pad, st).numpy()
    assert np.array_equal(y2, (2 * y).astype(np.float32))


def test_config5_wrn_block_step_matches_the_oracle():
    """One pre-activation block at a stage entry (stride 2, widths 16 -> 32, 1x1 projection shortcut
    from the block input), mean pool, dense, softmax, cross entropy and weight decay: gradients of
    every parameter against a hand-composed oracle pass, then one ADAM step."""
    n, cin, u, h = 8, 16, 32, 8
    g = np.random.default_rng(60)
    X = g.standard_normal((n, cin, h, h)).astype(np.float32)
    Y = workloads.one_hot(g.integers(0, 10, n))
    feats, labels = float32([n, cin, h, h]), float32([n, 10])
    init = nnet.Init(61)
    blk = nnet._wrn_block(nnet.dataSource(feats), u, 1, 2, init, 1e-4)
    head = nnet.softmax(nnet.dense(nnet.meanPool(nnet.relu(nnet.batchNorm(blk))), 10, init))
    net = nnet.DAGNetwork([feats], [head])
    loss = nnet.crossEntropy(head.trainOutput, labels) + net.paramLoss
    names = ["g1", "b1", "rm1", "rv1", "w1", "g2", "b2", "rm2", "rv2", "w2", "ws", "g3", "b3", "rm3", "rv3", "wd", "bd"]
    assert len(net.params) == len(names)
    P = {k: p.value.copy() for k, p in zip(names, net.params)}
    grads = grad(loss, net.params)
    got = core.evaluate([loss] + grads, {feats: X, labels: Y})

    # ---- oracle forward
    def bn(x, k):
        packed = O.bn_train(x, P["g" + k], P["b" + k], P["rm" + k], P["rv" + k], 0.9)
        return packed[:x.size].reshape(x.shape)
    a1 = bn(X, "1"); r1 = O.relu(a1)
    c1 = O.convolution(r1, P["w1"], (1, 1), (2, 2))
    a2 = bn(c1, "2"); r2 = O.relu(a2)
    c2 = O.convolution(r2, P["w2"], (1, 1), (1, 1))
    sc = O.convolution(X, P["ws"], (0, 0), (2, 2))
    s = (c2 + sc).astype(np.float32)
    a3 = bn(s, "3"); r3 = O.relu(a3)
    hw = r3.shape[2] * r3.shape[3]
    pooled = (r3.reshape(n * u, hw).astype(np.float64).sum(axis=1) * np.float32(1.0 / hw)).reshape(n, u).astype(np.float32)
    z = (pooled.astype(np.float64) @ P["wd"].astype(np.float64).T + P["bd"]).astype(np.float32)
    p = O.softmax(z, f64=True)
    decay = sum(1e-4 * (P[k].astype(np.float64) ** 2).sum() for k in ("w1", "w2", "ws"))
    want_loss = -(Y * np.log(p.astype(np.float64) + 1e-6)).sum() / n + decay
    assert_close(got[0], want_loss, "loss")

    # ---- oracle backward
    want = {}
    dp = (-(Y / (p.astype(np.float64) + 1e-6)) / n).astype(np.float32)
    dz = O.softmax_grad(dp, p)
    want["wd"] = dz.astype(np.float64).T @ pooled
    want["bd"] = dz.astype(np.float64).sum(axis=0)
    dpool = (dz.astype(np.float64) @ P["wd"]).astype(np.float32)
    dr3 = np.repeat((dpool * np.float32(1.0 / hw)).reshape(n, u, 1), hw, axis=2).reshape(r3.shape)

    def bn_back(dy, x, k):
        packed = O.bn_grad(dy, x, P["g" + k])
        c = x.shape[1]
        want["g" + k] = packed[x.size:x.size + c].reshape(P["g" + k].shape)
        want["b" + k] = packed[x.size + c:x.size + 2 * c]
        want["rm" + k] = np.zeros(c, np.float32)
        want["rv" + k] = np.zeros(c, np.float32)
        return packed[:x.size].reshape(x.shape)
    ds = bn_back(O.relu_grad(dr3, a3), s, "3")
    want["w2"] = O.conv_bwd_filter(ds, r2, P["w2"].shape, (1, 1), (1, 1)) + 2e-4 * P["w2"].astype(np.float64)
    dr2 = O.conv_bwd_data(ds, P["w2"], r2.shape, (1, 1), (1, 1))
    dc1 = bn_back(O.relu_grad(dr2, a2), c1, "2")
    want["w1"] = O.conv_bwd_filter(dc1, r1, P["w1"].shape, (1, 1), (2, 2)) + 2e-4 * P["w1"].astype(np.float64)
    want["ws"] = O.conv_bwd_filter(ds, X, P["ws"].shape, (0, 0), (2, 2)) + 2e-4 * P["ws"].astype(np.float64)
    dr1 = O.conv_bwd_data(dc1, P["w1"], r1.shape, (1, 1), (2, 2))
    bn_back(O.relu_grad(dr1, a1), X, "1")
    for k, gk in zip(names, got[1:]):
        assert_close(gk, np.asarray(want[k]).reshape(gk.shape), "gradient of " + k)

    # ---- one ADAM step moves every parameter with a gradient by ~alpha and replaces the running
    # statistics by the batch-norm outputs (projection), in both optimizer forms
    after = []
    for make in (online.adam, online.fused_adam):
        for k, prm in zip(names, net.params):
            prm.set_value(P[k])
        make([loss], net.params, net.paramProj)({feats: X, labels: Y})
        after.append([prm.value.copy() for prm in net.params])
    for k, a, b in zip(names, *after):
        assert np.array_equal(a, b), k
    rm1 = O.bn_train(X, P["g1"], P["b1"], P["rm1"], P["rv1"], 0.9)[X.size:X.size + cin]
    assert_close(after[0][names.index("rm1")], rm1, "running mean after the step")


def test_config5_small_wide_resnet_step_matches_the_cpu_evaluator():
    """The whole Wide-ResNet graph (nnet/models/wrn.d:56-219: strided stage entries, 1x1 projections from the
    block input, weight decay, mean pool as a GEMV) at depth 10, width 2, batch 4: loss, predictions and
    every parameter gradient from HIPPlan, with and without the rewrites, against the same graph on the CPU
    evaluator."""
    n = 4
    r = np.random.default_rng(70)
    X = r.standard_normal((n, 3, 32, 32)).astype(np.float32)
    Y = workloads.one_hot(r.integers(0, 10, n))
    feats, labels = float32([n, 3, 32, 32]), float32([n, 10])
    init = nnet.Init(71)
    preds = nnet.softmax(nnet.dense(nnet.wideResNet(feats, 10, 2, init), 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    grads = grad(loss, net.params)
    outs = [loss, preds.trainOutput] + grads
    want = evaluator.evaluate(outs, {feats: X, labels: Y})
    for flags in (0, configs.REWRITES):
        got = core.compile(outs, flags).execute({feats: X, labels: Y})
        for i, (g, w) in enumerate(zip(got, want)):
            assert_close(g, w, "output %d (%s), flags %d" % (i, outs[i].opType, flags))


def test_config5_wide_resnet_28_10_step_at_batch_128_rewrites_and_fused_update_change_nothing():
    """The full-size step through size-independent properties: every output of the plan with the rewrites on
    equals the plan without them bit for bit, and one fused ADAM step leaves the parameters the op-graph ADAM
    step leaves, bit for bit."""
    results = []
    for flags in (0, configs.REWRITES):
        step = configs.wide_resnet(128, fused=True, flags=flags)
        net, loss, preds = step.extra["net"], step.loss, step.extra["preds"]
        grads = grad(loss, net.params)
        plan = core.compile([loss, preds.trainOutput] + grads, flags)
        results.append(plan.execute(step.args))
        plan.cleanup()
        del step, plan
    for i, (a, b) in enumerate(zip(*results)):
        assert np.array_equal(a, b), i
    assert np.isfinite(results[0][0]) and all(np.isfinite(g).all() for g in results[0][2:])
    del results
    after = []
    for fused in (False, True):
        step = configs.wide_resnet(128, fused=fused, flags=configs.REWRITES)
        step.run(1)
        after.append((step.loss_value(), [p.value.copy() for p in step.params]))
        del step
    assert after[0][0] == after[1][0]
    for i, (a, b) in enumerate(zip(after[0][1], after[1][1])):
        assert np.array_equal(a, b), i


# ------------------------------------------------------------------------------ evaluation path
@pytest.mark.parametrize("flags", [0, core.PLAN_VIEWS | core.PLAN_FUSE])
def test_eval_plan_uses_running_statistics(flags):
    """examples/cifar10.d:84-87 compiles a second plan on the layers' `output` (batchNormInference,
    dropout scaled instead of sampled).  After a few training steps the running statistics differ from
    their initial values; the test plan must normalise with them, not with batch statistics."""
    init = nnet.Init(5)
    x, y = float32([16, 3, 8, 8]), float32([16, 10])
    l1 = nnet.relu(nnet.batchNorm(nnet.conv2D(nnet.dataSource(x), 8, (3, 3), init, padding=(1, 1))))
    l2 = nnet.dropout(nnet.maxPool(l1, (2, 2)), 0.25)
    top = nnet.softmax(nnet.dense(l2, 10, init))
    net = nnet.DAGNetwork([x], [top])
    loss = nnet.crossEntropy(top.trainOutput, y) + net.paramLoss
    r = np.random.default_rng(0)
    xs = r.standard_normal((16, 3, 8, 8)).astype(np.float32)
    ys = np.eye(10, dtype=np.float32)[r.integers(0, 10, 16)]
    up = online.fused_sgd([loss], net.params, net.paramProj, 0.05, flags=flags)
    for _ in range(4):
        up({x: xs, y: ys})
    w, b, gamma, beta, mean, var, wd, bd = [p.value for p in net.params]
    assert np.abs(mean).max() > 1e-3 and np.abs(var - 1).max() > 1e-3

    test_plan = core.compile([top.output], flags)
    xt = r.standard_normal((16, 3, 8, 8)).astype(np.float32)
    got, = test_plan.execute({x: xt})
    h = O.add_bias(O.convolution(xt, w, (1, 1), (1, 1)), b)
    h = O.relu(O.bn_infer(h, gamma.ravel(), beta, mean, var))
    h = O.maxpool(h, (2, 2)) * np.float32(0.75)
    z = (h.reshape(16, -1).astype(np.float64) @ wd.astype(np.float64).T + bd).astype(np.float32)
    assert_close(got, O.softmax(z, f64=True), "eval plan")
    assert np.array_equal(got, test_plan.execute({x: xt})[0])   # no sampling on the eval path
