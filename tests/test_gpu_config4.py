"""The headline workload as a parity case: the VGG-16-style CIFAR network with batch norm
(nnet/models/vgg.d:54-62,85-142 as examples/cifar10.d:64-66 uses it), FC 512-512-10, softmax cross
entropy, one SGD step.

  * batch 8: the whole step through HIPPlan, with and without the plan rewrites, against an oracle pass
    composed from the CPU oracle's operations: loss, predictions, every parameter gradient, all 26
    running statistics, and the parameters after one SGD step in both optimizer forms;
  * batch 128 (the benchmark's size): every convolution's forward and backward-data output on the
    first two and last two images against the float64 oracle run on just those images (images are
    independent), every filter gradient on a block of (output channel, input channel) pairs against
    the oracle run on just those channels (pairs are independent), batch norm and its gradient on the
    two large-channel layers and one register-resident layer, max-pooling and its gradient bit for bit,
    the dense head against float64 products -- all on the tensors the step itself produces
    (He-scaled weights, post-ReLU activations, real upstream gradients), at the stated tolerance
    rtol 1e-4 / atol 1e-5 without any rescaling;
  * batch 128: the step with the rewrites on against the step with the rewrites off, and fused against
    op-graph SGD after two steps, bit for bit.

The largest error seen per quantity is recorded (tests/util.py: err_ratio)."""
import numpy as np
import pytest

import oracle as O
from dopt_amd import core, nnet, online, ops, workloads
from dopt_amd.core import float32, grad
from util import err_ratio

pytestmark = pytest.mark.gpu

REWRITES = core.PLAN_VIEWS | core.PLAN_FUSE
MOMENTUM = float(np.float32(0.9))


def _vgg_net(batch, seed, sizes=nnet.VGG16_SIZES, dense=(512, 512)):
    feats, labels = float32([batch, 3, 32, 32]), float32([batch, 10])
    init = nnet.Init(seed)
    preds = nnet.softmax(nnet.dense(nnet.vgg(feats, sizes, list(dense), init), 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    return feats, labels, net, loss, preds


def _inputs(batch, seed):
    r = np.random.default_rng(seed)
    x = r.standard_normal((batch, 3, 32, 32)).astype(np.float32)
    y = workloads.one_hot(r.integers(0, 10, batch))
    return x, y


def _conv_layers(net):
    """(conv layer, batch-norm layer) pairs in network order."""
    out = []
    for i, layer in enumerate(net.layers):
        if layer.trainOutput.opType == "addBias" and layer.trainOutput.deps[0].opType == "convolution":
            out.append((layer, net.layers[i + 1]))
    return out


# --------------------------------------------------------------------------------- the oracle pass
def _vgg_oracle(X, Y, P, sizes, ndense, decide=None):
    """Forward, backward and the running-statistics update of the network, composed from the oracle's
    operations.  P: parameter values in network order.  Returns loss, predictions, the gradients in
    parameter order (None for the running statistics, which have no gradient), the new running
    statistics per batch-norm layer and the batch-norm outputs.

    `decide`: the device's batch-norm outputs, one per convolution layer.  Backward passes make discrete decisions
    from forward values - which activations a relu lets through, which element of a window a max-pool routes to - and
    two correct fp32 forward passes (a direct and a Winograd convolution differ by ~1e-6) can disagree about the sign of
    an activation that is zero to five digits, or about the larger of two values that agree to seven.  One such flip
    moves every gradient below it by ~1e-3 of its size.  And the forward difference itself grows from layer to layer
    (batch norm over the 32 values a channel has in the last layers at batch 8 amplifies what the layers below
    left): thirteen layers on, two correct passes differ by about the tolerance stated for ONE operation.  With
    `decide`, every layer of the oracle's pass therefore starts from the device's output of the layer below: its own
    batch-norm output (returned, and checked against the device's at the stated tolerance) is what that operation
    makes of the same input, the relu masks and pool positions of the backward pass are those of the values the
    device really had, and all arithmetic is still the oracle's."""
    n = X.shape[0]
    it = iter(P)
    a, tape, ys = X, [], []
    for s in sizes:
        if s == -1:
            tape.append(("pool", a))
            a = O.maxpool(a, (2, 2))
            continue
        w, b, gamma, beta, rm, rv = (next(it) for _ in range(6))
        c = O.convolution(a, w, (1, 1), (1, 1))
        cb = O.add_bias(c, b)
        packed = O.bn_train(cb, gamma.reshape(-1), beta, rm, rv, MOMENTUM)
        y = packed[:cb.size].reshape(cb.shape)
        k = cb.shape[1]
        tape.append(("conv", a, w, cb, gamma, y if decide is None else decide[len(ys)], packed[cb.size:cb.size + k],
                     packed[cb.size + k:]))
        a = O.relu(y if decide is None else decide[len(ys)])
        ys.append(y)
    feat_shape = a.shape
    a = a.reshape(n, -1)
    dense = []
    for i in range(ndense):
        W, b = next(it), next(it)
        z = (a.astype(np.float64) @ W.astype(np.float64).T + b).astype(np.float32)   # layers/dense.d:107,143
        dense.append((a, W, z))
        a = O.relu(z) if i < ndense - 1 else O.softmax(z, f64=True)
    p = a
    loss = -(Y * np.log(p.astype(np.float64) + 1e-6)).sum() / n                       # nnet/losses.d:23-26

    dp = (-(Y / (p.astype(np.float64) + 1e-6)) / n).astype(np.float32)
    dz = O.softmax_grad(dp, p)
    gdense = []
    for i in reversed(range(ndense)):
        a_in, W, z = dense[i]
        gdense.append((dz.astype(np.float64).T @ a_in.astype(np.float64), dz.astype(np.float64).sum(axis=0)))
        da = (dz.astype(np.float64) @ W.astype(np.float64)).astype(np.float32)
        if i:
            dz = O.relu_grad(da, dense[i - 1][2])
    gdense.reverse()
    d = da.reshape(feat_shape)
    gconv, stats = [], []
    for rec in reversed(tape):
        if rec[0] == "pool":
            d = O.maxpool_grad(d, rec[1], (2, 2))
            continue
        _, a_in, w, cb, gamma, y, new_mean, new_var = rec
        packed = O.bn_grad(O.relu_grad(d, y), cb, gamma.reshape(-1))
        k = cb.shape[1]
        dcb = packed[:cb.size].reshape(cb.shape)
        gconv.append((O.conv_bwd_filter(dcb, a_in, w.shape, (1, 1), (1, 1)), O.add_bias_grad(dcb),
                      packed[cb.size:cb.size + k].reshape(gamma.shape), packed[cb.size + k:], None, None))
        stats.append((new_mean, new_var))
        d = O.conv_bwd_data(dcb, w, a_in.shape, (1, 1), (1, 1))
    gconv.reverse()
    stats.reverse()
    grads = [g for block in gconv for g in block] + [g for pair in gdense for g in pair]
    return loss, p, grads, stats, ys


NAMES = ("filter", "bias", "gamma", "beta", "mean", "var")


def _param_name(i, nconv):
    if i < 6 * nconv:
        return "conv%d %s" % (i // 6 + 1, NAMES[i % 6])
    j = i - 6 * nconv
    return "dense%d %s" % (j // 2 + 1, "weight" if j % 2 == 0 else "bias")


@pytest.mark.parametrize("flags", [0, REWRITES], ids=["plain", "rewrites"])
def test_config4_whole_step_matches_the_oracle_at_batch_8(flags):
    batch, nconv = 8, 13
    X, Y = _inputs(batch, 40)
    feats, labels, net, loss, preds = _vgg_net(batch, 41)
    assert len(net.params) == 6 * nconv + 6 and len(net.paramProj) == 2 * nconv
    P0 = [p.value.copy() for p in net.params]
    grads = grad(loss, net.params)
    stat_params = [p for p in net.params if p in net.paramProj]
    bn_out = [bn.trainOutput for _, bn in _conv_layers(net)]
    assert len(bn_out) == nconv
    plan = core.compile([loss, preds.trainOutput] + grads + [net.paramProj[p](p) for p in stat_params] + bn_out, flags)
    got = plan.execute({feats: X, labels: Y})
    case = "config4 b8 step %s" % ("rewrites" if flags else "plain")
    dev_y = got[len(got) - nconv:]
    # every layer of the oracle's pass starts from the device's output of the layer below (see _vgg_oracle): what the
    # oracle makes of the same input is checked here, layer by layer, and its backward pass takes the relu / max-pool
    # decisions the device's forward values imply
    want_loss, want_p, want_g, want_stats, want_y = _vgg_oracle(X, Y, P0, nnet.VGG16_SIZES, 3, decide=dev_y)
    for j, (g, w) in enumerate(zip(dev_y, want_y)):
        assert err_ratio(g, w, "conv%d batch-norm output" % (j + 1), case) <= 1.0
    # every quantity at the stated tolerance (rtol 1e-4, atol 1e-5, no rescaling), although the backward chain is 13
    # blocks deep and what is compared is this backend's whole backward pass against the oracle's
    assert err_ratio(got[0], want_loss, "loss", case) <= 1.0
    assert err_ratio(got[1], want_p, "predictions", case) <= 1.0
    for i, (g, w) in enumerate(zip(got[2:2 + len(grads)], want_g)):
        name = _param_name(i, nconv)
        if w is None:
            assert not g.any(), name           # running statistics have no gradient
            continue
        # (a convolution bias in front of a batch norm has the exact gradient 0: both sides hold rounding
        # noise of sum(dx), far below atol)
        assert err_ratio(g, np.asarray(w).reshape(g.shape), "d " + name, case) <= 1.0, name
    k = 2 + len(grads)
    for j, (mean, var) in enumerate(want_stats):
        assert err_ratio(got[k + 2 * j], mean, "conv%d new running mean" % (j + 1), case) <= 1.0
        assert err_ratio(got[k + 2 * j + 1], var, "conv%d new running variance" % (j + 1), case) <= 1.0

    # one SGD step, op-graph form and fused kernel: identical parameters; w' = w - lr g to the bit with this
    # plan's own gradients, running statistics replaced by the batch-norm outputs
    after = []
    for make in (online.sgd, online.fused_sgd):
        for p, v in zip(net.params, P0):
            p.set_value(v)
        up = make([loss], net.params, net.paramProj, flags=flags)
        lv, = up({feats: X, labels: Y})
        assert lv == got[0]
        after.append([p.value.copy() for p in net.params])
    for i, (a, b) in enumerate(zip(*after)):
        name = _param_name(i, nconv)
        assert np.array_equal(a, b), name
        if want_g[i] is None:
            j, which = divmod(i, 6)
            assert np.array_equal(a, got[k + 2 * j + (which - 4)]), name
        else:
            step, _ = O.sgd_step(P0[i], got[2 + i].reshape(P0[i].shape), np.zeros_like(P0[i]), 0.01, 0.0)
            assert np.array_equal(a, step), name


# --------------------------------------------------------------------------------- batch 128, layer by layer
IMAGES = [0, 1, 126, 127]


def _pairs(k, c):
    ks = sorted({0, 1, k // 2, k - 2, k - 1})
    cs = sorted({0, 1, c // 2, c - 2, c - 1} & set(range(c)))
    return ks, cs


def test_config4_batch_128_layers_match_the_oracle_on_the_steps_own_tensors():
    batch = 128
    X, Y = _inputs(batch, 0)
    feats, labels, net, loss, preds = _vgg_net(batch, 1)
    layers = _conv_layers(net)
    assert len(layers) == 13
    relu_of = {id(l.deps[0]): l for l in net.layers if l.trainOutput.opType == "relu"}
    pools = [l for l in net.layers if l.trainOutput.opType == "maxpool"]
    head = [l for l in net.layers if l.params and l.params[0].symbol.rank == 2]
    assert len(pools) == 5 and len(head) == 3
    wanted = []           # intermediate values whose gradients the checks read
    for conv, bn in layers:
        wanted += [conv.deps[0].trainOutput, conv.trainOutput, bn.trainOutput, relu_of[id(bn)].trainOutput]
    wanted += [p.trainOutput for p in pools] + [l.trainOutput for l in head]
    gall = grad(loss, net.params + wanted[1:])            # (the input batch itself has no gradient)
    gparam = dict(zip(map(id, net.params), gall))
    ginter = dict(zip(map(id, wanted[1:]), gall[len(net.params):]))
    # flags 0: one kernel and one buffer per operation, every intermediate value stays readable
    plan = core.compile([loss, preds.trainOutput] + gall[:len(net.params)], 0)
    plan.execute({feats: ops.tensor(X), labels: ops.tensor(Y)}, [None] * len(plan.outputs))
    R = plan.result
    case = "config4 b128 layer"
    P = {id(p): p.value for p in net.params}

    for li, (conv, bn) in enumerate(layers):
        tag = "conv%d" % (li + 1)
        x_op, cb_op, y_op = conv.deps[0].trainOutput, conv.trainOutput, bn.trainOutput
        c_op = cb_op.deps[0]
        w_sym, b_sym = conv.params[0].symbol, conv.params[1].symbol
        w, b = P[id(w_sym)], P[id(b_sym)]
        x, c = (X if li == 0 else R(x_op)), R(c_op)
        dcb = R(ginter[id(cb_op)])                       # gradient of addBias's output = of the convolution's
        # C1 on four images
        want = O.convolution(x[IMAGES], w, (1, 1), (1, 1))
        assert err_ratio(c[IMAGES], want, tag + " convolution", case) <= 1.0
        # C2 on four images (the first layer's input needs no gradient: the plan never computes it)
        if li > 0:
            dx = R(ginter[id(x_op)])
            want = O.conv_bwd_data(dcb[IMAGES], w, x[IMAGES].shape, (1, 1), (1, 1))
            assert err_ratio(dx[IMAGES], want, tag + " convolutionFeaturesGrad", case) <= 1.0
        # C3 on a block of (k, c) pairs over the whole batch
        dw = R(gparam[id(w_sym)])
        ks, cs = _pairs(w.shape[0], w.shape[1])
        want = O.conv_bwd_filter(np.ascontiguousarray(dcb[:, ks]), np.ascontiguousarray(x[:, cs]),
                                 (len(ks), len(cs), 3, 3), (1, 1), (1, 1))
        assert err_ratio(dw[np.ix_(ks, cs)], want, tag + " convolutionFiltersGrad", case) <= 1.0
        # A3 / A4
        cb = R(cb_op)
        assert np.array_equal(cb, O.add_bias(c, b)), tag
        db = R(gparam[id(b_sym)])
        err_ratio(db, O.add_bias_grad(dcb), tag + " addBiasGrad", case)
        assert np.abs(db).max() <= 1e-5, tag             # its exact value is 0: in front of a batch norm
        # B1 / B2 (+ A1 / A2 around them) on the two large-channel layers and two register-resident ones
        if li in (0, 1, 3, 9):
            g_sym, be_sym, rm_sym, rv_sym = (q.symbol for q in bn.params)
            gamma = P[id(g_sym)].reshape(-1)
            y = R(y_op)
            packed = O.bn_train(cb, gamma, P[id(be_sym)], P[id(rm_sym)], P[id(rv_sym)], MOMENTUM)
            assert err_ratio(y, packed[:cb.size], tag + " batchNormTrain y", case) <= 1.0
            r_op = relu_of[id(bn)].trainOutput
            assert np.array_equal(R(r_op), O.relu(y)), tag
            dy_bn = R(ginter[id(y_op)])
            assert np.array_equal(dy_bn, O.relu_grad(R(ginter[id(r_op)]), y)), tag
            gp = O.bn_grad(dy_bn, cb, gamma)
            k = cb.shape[1]
            assert err_ratio(dcb, gp[:cb.size], tag + " batchNormGrad dx", case) <= 1.0
            assert err_ratio(R(gparam[id(g_sym)]), gp[cb.size:cb.size + k], tag + " batchNormGrad dscale", case) <= 1.0
            assert err_ratio(R(gparam[id(be_sym)]), gp[cb.size + k:], tag + " batchNormGrad dbias", case) <= 1.0

    # M1 / M2 bit for bit on every pooling layer
    for pi, pool in enumerate(pools):
        xin_op = pool.deps[0].trainOutput
        xin = R(xin_op)
        assert np.array_equal(R(pool.trainOutput), O.maxpool(xin, (2, 2))), pi
        want = O.maxpool_grad(R(ginter[id(pool.trainOutput)]), xin, (2, 2))
        assert np.array_equal(R(ginter[id(xin_op)]), want), pi

    # dense head: G1 and its two gradients on the step's own activations
    for di, layer in enumerate(head):
        w_sym = layer.params[0].symbol
        W = P[id(w_sym)]
        mm = layer.trainOutput.deps[0]                   # matmul(x, transpose(W)), layers/dense.d:107
        assert mm.opType == "matmul"
        a = R(mm.deps[0])
        tag = "dense%d" % (di + 1)
        assert err_ratio(R(mm), a.astype(np.float64) @ W.astype(np.float64).T, tag + " matmul", case) <= 1.0
        dz = R(ginter[id(layer.trainOutput)])
        want = dz.astype(np.float64).T @ a.astype(np.float64)
        assert err_ratio(R(gparam[id(w_sym)]), want, tag + " weight gradient", case) <= 1.0
        want = dz.astype(np.float64).sum(axis=0)
        assert err_ratio(R(gparam[id(layer.params[1].symbol)]), want, tag + " bias gradient", case) <= 1.0
    plan.cleanup()


def test_config4_batch_128_rewrites_and_fused_update_change_nothing():
    batch, nconv = 128, 13
    X, Y = _inputs(batch, 0)
    tx, ty = ops.tensor(X), ops.tensor(Y)
    results = []
    for flags in (0, REWRITES):
        feats, labels, net, loss, preds = _vgg_net(batch, 1)
        grads = grad(loss, net.params)
        stat_params = [p for p in net.params if p in net.paramProj]
        plan = core.compile([loss, preds.trainOutput] + grads + [net.paramProj[p](p) for p in stat_params], flags)
        results.append(plan.execute({feats: tx, labels: ty}))
        plan.cleanup()
    differing = []
    for i, (a, b) in enumerate(zip(*results)):
        if not np.array_equal(a, b):
            differing.append(i)
            # only the bias gradient of a convolution in front of a batch norm: the fused kernel sums dx in
            # another order, and the exact value is 0
            name = _param_name(i - 2, nconv)
            assert name.startswith("conv") and name.endswith("bias"), name
            assert max(np.abs(a).max(), np.abs(b).max()) <= 1e-5, name
    assert len(differing) <= nconv

    # fused SGD against the op-graph SGD, two steps, with the rewrites on (what the benchmark runs)
    after = []
    for make in (online.sgd, online.fused_sgd):
        feats, labels, net, loss, preds = _vgg_net(batch, 1)
        up = make([loss], net.params, net.paramProj, flags=REWRITES)
        losses = [up({feats: tx, labels: ty})[0] for _ in range(2)]
        after.append((losses, [p.value.copy() for p in net.params]))
        del up
    assert after[0][0] == after[1][0] and after[0][0][0] == results[1][0]
    for i, (a, b) in enumerate(zip(after[0][1], after[1][1])):
        assert np.array_equal(a, b), _param_name(i, nconv)
    assert np.isfinite(after[0][0]).all() and after[0][0][1] != after[0][0][0]
