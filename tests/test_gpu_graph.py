"""The backend behind its plugin boundary: graphs built with the reference's op constructors,
executed by HIPPlan through the C ABI.  Replays every known-answer test the reference holds
(they all go through `evaluate`), the registry contract, plan semantics, and the optimizers
(op-graph form vs fused kernels vs the oracle)."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from util import assert_close

pytestmark = pytest.mark.gpu

from dopt_amd import core
from dopt_amd import capi, configs, nnet, online, ops, workloads  # noqa: E402
from dopt_amd.core import (evaluate, float32, float32Constant, grad, int32)  # noqa: E402


def _f(shape, vals):
    return float32(shape, np.array(vals, np.float32))


# ----------------------------------------------------------------------------- reference KATs through evaluate()
def test_kat_slice_pad_reshape_transpose_repeat(kats):
    k = kats["slice"]
    out = evaluate(core.slice(int32(k["shape"], k["input"]), k["start"], k["stop"]))
    assert out.dtype == np.int32 and out.ravel().tolist() == k["expected"]
    k = kats["pad"]
    assert evaluate(core.pad(int32(k["shape"], k["input"]), k["before"], k["after"])).ravel().tolist() == k["expected"]
    k = kats["reshape"]
    r1 = _f(k["shape"], k["input"]).reshape(k["newShape"])
    assert r1.shape == tuple(k["newShape"]) and evaluate(r1).ravel().tolist() == k["expected"]
    k = kats["transpose"]
    assert evaluate(core.transpose(_f(k["shape"], k["input"]), k["order"])).ravel().tolist() == k["expected"]
    for name in ("repeat_1x1", "repeat_2x2"):
        k = kats[name]
        got = evaluate(core.repeat(_f(k["shape"], k["input"]), k["repetitions"]))
        assert got.ravel().tolist() == [float(v) for v in k["expected"]]
    k = kats["repeat_scalar_count"]
    assert evaluate(core.repeat(_f(k["shape"], k["input"]), k["repetitions"])).ravel().tolist() == k["expected"]


def test_kat_matmul_sum_argmin_max(kats):
    k = kats["matmul"]
    assert evaluate(core.matmul(_f(k["a_shape"], k["a"]), _f(k["b_shape"], k["b"]))).ravel().tolist() == k["expected"]
    for c in kats["sum"]["cases"]:
        assert evaluate(core.sum(_f(c["shape"], c["input"]), c["axes"])).ravel().tolist() == c["expected"]
    for c in kats["argmin"]["cases"]:
        out = evaluate(core.argmin(_f(c["shape"], c["input"]), c["axis"]))
        assert out.dtype == np.int32 and out.ravel().tolist() == c["expected"]
    for c in kats["maxElement"]["cases"]:
        assert evaluate(core.maxElement(_f(c["shape"], c["input"]), c["axes"])).ravel().tolist() == c["expected"]


def test_kat_convolution_maxpool_softmax(kats):
    k = kats["convolution"]
    y = evaluate(core.convolution(_f(k["features_shape"], k["features"]), _f(k["filters_shape"], k["filters"])))
    assert y.ravel().tolist() == [float(v) for v in k["expected"]]       # pins the filter flip
    k = kats["maxpool"]
    assert evaluate(core.maxpool(_f(k["shape"], k["input"]), k["dims"])).ravel().tolist() == \
        [float(np.float32(v)) for v in k["expected"]]
    k = kats["softmax"]
    assert np.allclose(evaluate(core.softmax(_f(k["shape"], k["input"]))).ravel(), k["expected"], rtol=k["rel"],
                       atol=k["abs"])


def test_kat_grads_and_scalar_plan(kats):
    x = float32()
    y = x * x
    r = np.float32(-63.21875)
    g = evaluate(grad(y, [x]), {x: np.array([r])})[0]
    assert g[()] == r + r                                                 # grads/package.d:113-129
    k = kats["slice_grad"]
    a, b = _f(k["shape"], k["a"]), _f(k["shape"], k["b"])
    c = core.slice(a * b, k["start"], k["stop"])
    assert evaluate(grad(c, [a]))[0].ravel().tolist() == [float(v) for v in k["expected"]]
    k = kats["scalar_plan"]
    assert evaluate(_f([], [k["a"]]) * _f([], [k["b"]]) + _f([], [k["c"]]))[()] == k["expected"]


def test_kat_batchnorm_running_mean_with_adam(kats):
    # nnet/layers/batchnorm.d:158-177, through the op-graph ADAM and the projections
    k = kats["batchnorm_running_mean"]
    x = _f(k["shape"], k["x"])
    layers = nnet.batchNorm(nnet.dataSource(x))
    net = nnet.DAGNetwork([x], [layers])
    trloss = core.sum(layers.trainOutput)
    updater = online.adam([trloss], net.params, net.paramProj)
    for _ in range(200):                      # 0.9^200 ~ 7e-10: converged far below the 1e-2 tolerance
        updater.step_async(None)
    mean = layers.params[2].symbol.value
    assert np.allclose(mean, k["expected_running_mean"], rtol=k["rel"], atol=k["abs"])


# ----------------------------------------------------------------------------- registry (cuda/package.d:479-507)
def test_registry_contract():
    names = core.list_operations()
    for n in ["add", "matmul", "convolution", "convolutionFeaturesGrad", "convolutionFiltersGrad", "maxpool",
              "maxpoolGrad", "softmax", "softmaxGrad", "relu", "reluGrad", "addBias", "addBiasGrad", "batchNormTrain",
              "batchNormGrad", "batchNormInference", "slice", "pad", "repeat", "transpose", "sum", "maxElement",
              "argmin", "variable", "reshape"]:
        assert n in names, n
    lib = core._lib()
    CTOR = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p)
    ctor = CTOR(lambda g, op, user, out: 1)
    rc = lib.dopt_hip_register_kernel(b"add", C.cast(ctor, C.c_void_p), None)
    assert rc == 1 and b"already registered" in lib.dopt_hip_last_error()
    # deregister then the op cannot be planned; re-registering a refusing constructor also fails loudly
    assert lib.dopt_hip_deregister_kernel(b"atanh") == 0
    assert "atanh" not in core.list_operations()
    with pytest.raises(capi.HipError, match="Could not construct a HIP kernel"):
        evaluate(core.atanh(_f([2], [0.5, -0.5])))
    assert lib.dopt_hip_register_kernel(b"atanh", C.cast(ctor, C.c_void_p), None) == 0
    with pytest.raises(capi.HipError, match="Could not construct a HIP kernel"):
        evaluate(core.atanh(_f([2], [0.5, -0.5])))
    lib.dopt_hip_deregister_kernel(b"atanh")


def test_custom_kernel_through_the_registry():
    lib = core._lib()

    class Kernel(C.Structure):
        _fields_ = [("self", C.c_void_p), ("execute", C.c_void_p), ("destroy", C.c_void_p)]

    EXEC = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.c_void_p,
                       C.c_size_t)
    CTOR = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(Kernel))
    calls = []

    def execute(self, nin, inputs, nbytes, out, out_bytes):
        calls.append((nin, nbytes[0], out_bytes))
        # an "atanh" that is really a device-to-device copy of its input
        return capi.load().dopt_hip_copy_d2d(out, inputs[0], out_bytes)
    exec_c = EXEC(execute)

    def ctor(graph, op, user, out):
        out[0].self = None
        out[0].execute = C.cast(exec_c, C.c_void_p)
        out[0].destroy = None
        return 0
    ctor_c = CTOR(ctor)
    lib.dopt_hip_deregister_kernel(b"atanh")
    assert lib.dopt_hip_register_kernel(b"atanh", C.cast(ctor_c, C.c_void_p), None) == 0
    try:
        got = evaluate(core.atanh(_f([3], [5, -7, 0])))
        assert got.tolist() == [5.0, -7.0, 0.0] and calls == [(1, 12, 12)]
    finally:
        lib.dopt_hip_deregister_kernel(b"atanh")


# ----------------------------------------------------------------------------- plan semantics
def test_plan_args_must_be_variables_and_sizes_must_match():
    a = _f([2], [1, 2])
    y = a + a
    plan = core.compile([y])
    with pytest.raises(capi.HipError, match="opType of 'variable'"):
        plan.execute({y: np.zeros(2, np.float32)})
    with pytest.raises(capi.HipError):
        plan.execute({a: np.zeros(3, np.float32)})
    assert plan.execute({a: np.array([3, 4], np.float32)})[0].tolist() == [6.0, 8.0]
    assert plan.execute()[0].tolist() == [2.0, 4.0]          # falls back to the variable's own value
    plan.cleanup()


def test_plan_views_do_not_change_results():
    r = np.random.default_rng(3)
    x = float32([4, 6, 5, 5], r.standard_normal((4, 6, 5, 5)).astype(np.float32))
    gamma = float32([1, 6, 1, 1], np.ones(6, np.float32))
    beta, mean = float32([6]), float32([6])
    var = float32([6], np.ones(6, np.float32))
    y, nm, nv = core.batchNormTrain(x, gamma, beta, mean, var, 0.9)
    loss = core.sum(core.relu(y) * core.relu(y))
    outs = [loss, nm, nv] + grad(loss, [x, gamma, beta])
    plain = core.compile(outs)
    views = core.compile(outs, core.PLAN_VIEWS)
    assert views.stats()["kernels"] < plain.stats()["kernels"]
    for a, b in zip(plain.execute(), views.execute()):
        assert np.array_equal(a, b)
    plain.cleanup()
    views.cleanup()


# ----------------------------------------------------------------------------- optimizers
def _toy_problem(seed):
    r = np.random.default_rng(seed)
    x = float32([16, 12], r.standard_normal((16, 12)).astype(np.float32))
    t = float32([16, 5], r.standard_normal((16, 5)).astype(np.float32))
    w = float32([12, 5], (r.standard_normal((12, 5)) * 0.3).astype(np.float32))
    b = float32([5], r.standard_normal(5).astype(np.float32))
    pred = core.matmul(x, w) + core.repeat(b, 16)
    loss = nnet.squaredError(pred, t)
    return loss, [w, b]


@pytest.mark.parametrize("rule", ["sgd", "nesterov", "adam", "amsgrad"])
def test_fused_updaters_match_the_op_graph_form_bit_for_bit(rule):
    loss_a, wrt_a = _toy_problem(5)
    loss_b, wrt_b = _toy_problem(5)
    if rule in ("sgd", "nesterov"):
        nest = rule == "nesterov"
        ua = online.sgd([loss_a], wrt_a, None, _f([], [0.05]), _f([], [0.9]), nest)
        ub = online.fused_sgd([loss_b], wrt_b, None, 0.05, 0.9, nest)
    else:
        ua = getattr(online, rule)([loss_a], wrt_a, None, _f([], [0.01]))
        ub = getattr(online, "fused_" + rule)([loss_b], wrt_b, None, 0.01)
    for step in range(5):
        la, lb = ua()[0], ub()[0]
        assert la == lb, (step, la, lb)
        for pa, pb in zip(wrt_a, wrt_b):
            assert np.array_equal(pa.value, pb.value), (rule, step)
    if rule in ("adam", "amsgrad"):
        assert np.array_equal(ua.means[0].value, ub.state["m"][0].numpy())
        assert np.array_equal(ua.vars[1].value, ub.state["v"][1].numpy())
        assert ua.b1.value[()] == np.float32(ub.opt.b1.value) and ua.b2.value[()] == np.float32(ub.opt.b2.value)
    if rule == "amsgrad":
        assert np.array_equal(ua.varhats[0].value, ub.state["vhat"][0].numpy())


@pytest.mark.parametrize("rule", ["sgd", "adam", "amsgrad"])
def test_fit_line_scenario(rule):
    # online/{sgd,adam,amsgrad}.d unittests: y = 3x + 2, one sample per step (the reference only prints m, c)
    r = np.random.default_rng(7)
    xs = r.uniform(-10, 10, 100).astype(np.float32)
    ys = np.float32(3) * xs + np.float32(2)
    x, m, c, y = float32(), float32(), float32(), float32()
    yhat = m * x + c
    obj = (yhat - y) * (yhat - y)
    if rule == "sgd":
        up, steps = online.sgd([obj], [m, c], None, _f([], [0.001]), _f([], [0.9])), 300
    else:
        up, steps = getattr(online, rule)([obj], [m, c], None, _f([], [0.1])), 1500
    for i in range(steps):
        up.step_async({x: xs[i % 100:i % 100 + 1], y: ys[i % 100:i % 100 + 1]})
    assert abs(m.value[()] - 3) < 0.1 and abs(c.value[()] - 2) < 0.5, (m.value, c.value)


# ----------------------------------------------------------------------------- config 1: softmax regression step
def test_config1_softmax_regression_step_matches_the_oracle():
    # examples/mnistlogit.d:39-47: softmax built by hand from matmul/maxElement/exp/sum/repeat/div, SGD lr 0.1
    r0, r1 = np.random.default_rng(0), np.random.default_rng(1)
    X = r0.random((100, 784)).astype(np.float32)
    lab = r1.integers(0, 10, 100)
    Y = np.zeros((100, 10), np.float32)
    Y[np.arange(100), lab] = 1
    feats, labels = float32([100, 784]), float32([100, 10])
    W, b = float32([784, 10]), float32([10])
    linear = core.matmul(feats, W) + core.repeat(b, 100)
    numer = core.exp(linear - core.maxElement(linear))
    denom = core.repeat(core.sum(numer, [1]).reshape([100, 1]), [1, 10])
    preds = numer / denom
    loss = nnet.crossEntropy(preds, labels)
    up = online.sgd([loss, preds], [W, b], None, _f([], [0.1]))
    loss0, p0 = up({feats: X, labels: Y})
    # zero weights: uniform predictions, loss = -log(0.1 + 1e-6)
    assert np.allclose(p0, 0.1, rtol=1e-6)
    assert_close(loss0, -np.log(0.1 + 1e-6), "initial loss")
    # oracle step: dL/dlinear = (softmax - Y)/100 for the composed graph; W' = W - 0.1 * X^T dlin
    dlin = (np.full((100, 10), 0.1) - Y) / 100.0 * (0.1 / (0.1 + 1e-6))
    assert_close(W.value, -0.1 * (X.astype(np.float64).T @ dlin), "W after one step", scale=0.01)
    assert_close(b.value, -0.1 * dlin.sum(axis=0), "b after one step", scale=0.01)
    loss1, _ = up({feats: X, labels: Y})
    assert loss1 < loss0


# ----------------------------------------------------------------------------- fused kernels
def test_fused_entry_points_equal_the_separate_kernels():
    r = np.random.default_rng(80)
    for shape, wshape in [((4, 16, 8, 8), (40, 16, 3, 3)), ((2, 8, 32, 32), (16, 8, 3, 3)), ((3, 6, 5, 7), (4, 6, 3, 3)),
                          ((64, 32, 2, 2), (48, 32, 3, 3))]:
        x = ops.tensor(r.standard_normal(shape).astype(np.float32))
        w = ops.tensor(r.standard_normal(wshape).astype(np.float32))
        b = ops.tensor(r.standard_normal(wshape[0]).astype(np.float32))
        want = ops.add_bias(ops.convolution(x, w, (1, 1)), b).numpy()
        got = ops.convolution_bias(x, w, b, (1, 1)).numpy()
        assert np.array_equal(got, want), shape
    for shape in [(8, 6, 4, 4), (40, 4, 32, 32), (16, 5, 3, 3), (128, 32, 2, 2)]:
        c = shape[1]
        x = ops.tensor((r.standard_normal(shape) + 0.5).astype(np.float32))
        g, bb, rm = (ops.tensor(r.standard_normal(c).astype(np.float32)) for _ in range(3))
        rv = ops.tensor((r.random(c) + 0.5).astype(np.float32))
        dy = ops.tensor(r.standard_normal(shape).astype(np.float32))
        n = x.size
        plain = ops.bn_train(x, g, bb, rm, rv, 0.9)
        y = ops.relu(plain.view(0, shape))
        fused = ops.bn_train_relu(x, g, bb, rm, rv, 0.9)
        assert np.array_equal(fused.numpy()[:n], y.numpy().reshape(-1)), shape
        assert np.array_equal(fused.numpy()[n:], plain.numpy()[n:]), shape
        want = ops.bn_grad(ops.relu_grad(dy, plain.view(0, shape)), x, g).numpy()
        got = ops.bn_grad_relu(dy, y, x, g).numpy()
        assert np.array_equal(got, want), shape


def test_plan_fusion_does_not_change_results():
    r = np.random.default_rng(81)
    X = r.standard_normal((8, 3, 8, 8)).astype(np.float32)
    Y = np.zeros((8, 10), np.float32)
    Y[np.arange(8), r.integers(0, 10, 8)] = 1
    results, kernels = [], []
    for flags in (0, core.PLAN_VIEWS, core.PLAN_VIEWS | core.PLAN_FUSE):
        feats, labels = float32([8, 3, 8, 8]), float32([8, 10])
        init = nnet.Init(82)
        body = nnet.vgg(feats, [16, 16, -1, 32, -1], [24], init)
        preds = nnet.softmax(nnet.dense(body, 10, init))
        net = nnet.DAGNetwork([feats], [preds])
        loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
        grads = core.grad(loss, net.params)
        plan = core.compile([loss, preds.trainOutput] + grads + [net.paramProj[p](p) for p in net.paramProj], flags)
        results.append(plan.execute({feats: X, labels: Y}))
        kernels.append(plan.stats()["kernels"])
    differing = 0
    for a, b, c in zip(*results):
        assert np.array_equal(a, b)
        if not np.array_equal(a, c):
            # only the bias gradient of a convolution feeding a batch norm may differ: the fused kernel
            # sums dx in another order.  Its exact value is 0 (a bias before a batch norm has no effect),
            # so both are rounding noise of the dx sum.
            assert a.ndim == 1 and np.allclose(a, c, rtol=0, atol=2e-5), (a, c)
            differing += 1
    assert differing <= 3
    # three conv blocks each lose addBias, relu, reluGrad and addBiasGrad as separate kernels, and the
    # two dense layers lose their transposes
    assert kernels[2] <= kernels[1] - 12 - 8, kernels


def test_pools_ride_in_the_batch_norm_kernels():
    """With the rewrites on, the 2 x 2 max-pools of a VGG block and their gradients have no kernels of their
    own: the batch norm in front pools, the batch-norm gradient routes.  (That the values do not change is the
    test above and the configuration tests; this one checks that the rewrite really fires.)  The two
    convolutions behind the first pool run on 16 x 16 images, where backward-data takes a packed filter: each shares
    one step with its filter gradient."""
    r = np.random.default_rng(83)
    X = r.standard_normal((8, 3, 32, 32)).astype(np.float32)
    Y = np.zeros((8, 10), np.float32)
    Y[np.arange(8), r.integers(0, 10, 8)] = 1
    feats, labels = float32([8, 3, 32, 32]), float32([8, 10])
    init = nnet.Init(84)
    body = nnet.vgg(feats, [16, -1, 32, 32, -1], [24], init)
    preds = nnet.softmax(nnet.dense(body, 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    outs = [loss] + core.grad(loss, net.params)
    plan = core.compile(outs, core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_TIMING)
    fused = plan.execute({feats: X, labels: Y})
    prof = plan.profile()
    assert prof["batchNormTrain+relu+maxpool"][1] == 2, prof
    assert prof["maxpoolGrad+reluGrad+batchNormGrad+addBiasGrad"][1] == 2, prof
    assert "maxpool" not in prof and "maxpoolGrad" not in prof, prof
    assert prof["convolutionFeaturesGrad+convolutionFiltersGrad"][1] == 2 and "convolutionFeaturesGrad" not in prof, prof
    plain = core.compile(outs, core.PLAN_VIEWS).execute({feats: X, labels: Y})
    for a, b in zip(plain, fused):
        assert np.array_equal(a, b) or (a.ndim == 1 and np.allclose(a, b, rtol=0, atol=2e-5))


def test_backward_pair_waits_for_a_feature_operand_computed_in_between():
    """A graph written by hand in which the x operand of the filter gradient is itself computed, and only the filter
    gradient leads to it: in the plan's order it stands between backward-data and the filter gradient, so the two
    must not share a step placed where backward-data stands (the step would read x before it exists).  With the
    operand computed ahead of both, the same couple does share a step.  Values are those of the plain plan."""
    r = np.random.default_rng(1259)
    xs, k = (16, 128, 8, 8), 256
    X = r.standard_normal(xs).astype(np.float32)
    W = (r.standard_normal((k, xs[1], 3, 3)) * 0.05).astype(np.float32)
    DY = r.standard_normal((xs[0], k, xs[2], xs[3])).astype(np.float32)
    xv, wv, dyv = float32(list(xs)), float32(list(W.shape)), float32(list(DY.shape))
    args = {xv: X, wv: W, dyv: DY}
    flags = core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_TIMING
    # x computed between the two: two steps
    xc = core.relu(xv)
    dx = core.convolutionFeaturesGrad(dyv, wv, list(xs), [1, 1], [1, 1])
    dw = core.convolutionFiltersGrad(dyv, xc, list(W.shape), [1, 1], [1, 1])
    plan = core.compile([dx, dw], flags)
    got = plan.execute(args)
    prof = plan.profile()
    assert "convolutionFeaturesGrad+convolutionFiltersGrad" not in prof, prof
    want = core.compile([dx, dw], 0).execute(args)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    assert np.abs(want[1]).max() > 0
    # the same operand reached first (it is also an output ahead of the two): one step
    plan = core.compile([xc, dx, dw], flags)
    got = plan.execute(args)
    assert plan.profile()["convolutionFeaturesGrad+convolutionFiltersGrad"][1] == 1
    assert np.array_equal(got[1], want[0]) and np.array_equal(got[2], want[1])
    # the filter gradient first in the order: its step takes backward-data along (dy and the filter are ready)
    plan = core.compile([dw, dx], flags)
    got = plan.execute(args)
    assert plan.profile()["convolutionFeaturesGrad+convolutionFiltersGrad"][1] == 1
    assert np.array_equal(got[0], want[1]) and np.array_equal(got[1], want[0])


def test_packed_filter_entry_points_match_the_unpacked_ones():
    """dopt_hip_conv_pack_batch + the *_packed entry points against dopt_hip_conv_fwd_bias /
    dopt_hip_conv_bwd_data (themselves checked against the oracle in test_gpu_ops.py): same kernels,
    same packed layout, so the results are identical."""
    import ctypes as C
    from dopt_amd import capi
    lib = capi.load()
    r = np.random.default_rng(0)
    cases = [((4, 16, 8, 8), 32), ((2, 64, 32, 32), 64), ((8, 128, 4, 4), 256), ((16, 48, 2, 2), 40), ((3, 3, 16, 16), 8),
             ((2, 32, 16, 16), 96), ((20, 64, 2, 2), 128)]   # the last: 2 x 2 images read straight from the filter
    descs, flags, ws, packed, shapes = [], [], [], [], []
    for xs, k in cases:
        for bwd in (0, 1):
            d = ops.conv_desc(xs, (k, xs[1], 3, 3), (1, 1), (1, 1))
            nbytes = lib.dopt_hip_conv_packed_bytes(C.byref(d), bwd)
            if nbytes == 0:            # this shape and direction runs on the generic kernel
                continue
            assert nbytes % 4 == 0
            shapes.append((xs, k))
            w = ops.tensor(r.standard_normal((k, xs[1], 3, 3)).astype(np.float32))
            buf = ops.Tensor([nbytes // 4])
            descs.append(d); flags.append(bwd); ws.append(w); packed.append(buf)
    n = len(descs)
    assert n >= 6
    capi.check(lib.dopt_hip_conv_pack_batch(n, (type(descs[0]) * n)(*descs), (C.c_int * n)(*flags),
                                            (C.c_void_p * n)(*[w.ptr for w in ws]), (C.c_void_p * n)(*[b.ptr for b in packed])))
    for i, (xs, k) in enumerate(shapes):
        d, bwd, w, buf = descs[i], flags[i], ws[i], packed[i]
        ys = (xs[0], k, xs[2], xs[3])
        if not bwd:
            x = ops.tensor(r.standard_normal(xs).astype(np.float32))
            b = ops.tensor(r.standard_normal(k).astype(np.float32))
            want = ops.convolution_bias(x, w, b, (1, 1), (1, 1)).numpy()
            got = ops.Tensor(ys)
            capi.check(lib.dopt_hip_conv_fwd_bias_packed(C.byref(d), x.ptr, buf.ptr, b.ptr, got.ptr))
            assert np.array_equal(got.numpy(), want)
            capi.check(lib.dopt_hip_conv_fwd_bias_packed(C.byref(d), x.ptr, buf.ptr, None, got.ptr))
            assert np.array_equal(got.numpy(), ops.convolution(x, w, (1, 1), (1, 1)).numpy())
        else:
            dy = ops.tensor(r.standard_normal(ys).astype(np.float32))
            want = ops.conv_bwd_data(dy, w, xs, (1, 1), (1, 1)).numpy()
            got = ops.Tensor(xs)
            capi.check(lib.dopt_hip_conv_bwd_data_packed(C.byref(d), dy.ptr, buf.ptr, got.ptr))
            assert np.array_equal(got.numpy(), want)
    # shapes the patch kernels do not take report 0 and are refused by the packed entry points
    d5 = ops.conv_desc((2, 8, 8, 8), (8, 8, 5, 5), (2, 2), (1, 1))
    assert lib.dopt_hip_conv_packed_bytes(C.byref(d5), 0) == 0
    ds = ops.conv_desc((2, 16, 8, 8), (8, 16, 3, 3), (1, 1), (2, 2))
    assert lib.dopt_hip_conv_packed_bytes(C.byref(ds), 1) == 0
    x, y, scratch = ops.Tensor((2, 8, 8, 8)), ops.Tensor((2, 8, 8, 8)), ops.Tensor([1024])
    with pytest.raises(capi.HipError):
        capi.check(lib.dopt_hip_conv_fwd_bias_packed(C.byref(d5), x.ptr, scratch.ptr, None, y.ptr))


@pytest.mark.parametrize("xs,k", [((8, 256, 4, 4), 512),     # Winograd backward-data + filter gradient: 4 x 4 images, reductions split
                                  ((16, 128, 8, 8), 256),    # the same on rows of 8 pixels
                                  ((128, 128, 16, 16), 128), # ... at a benchmark shape
                                  ((8, 200, 4, 4), 512),     # one launch (200 rows would pad 64-row Winograd tiles by more than a fifth): 4 x 4 images, both reductions split
                                  ((16, 200, 8, 8), 256),    # one launch: rows of 8 pixels
                                  ((4, 200, 16, 16), 240),   # one launch, ragged: partial tiles in both products
                                  ((4, 160, 16, 16), 128),   # 160 input channels run as padded 64-row Winograd tiles: two launches
                                  ((2, 64, 32, 32), 64),     # 64-row tiles: the two kernels one after the other
                                  ((4, 64, 16, 16), 128),
                                  ((16, 48, 2, 2), 40)])     # dense 2x2 route
def test_backward_data_and_filter_gradient_as_one_call(xs, k):
    """dopt_hip_conv_bwd_pair_packed_open against dopt_hip_conv_bwd_data_packed + dopt_hip_conv_bwd_filter (checked
    against the oracle in test_gpu_ops.py): the same tiles in the same order, whether they run as one launch or two,
    so dx and dw are identical to the last bit; an open dx is closed by the batch-norm gradient or by
    dopt_hip_split_sum_close."""
    import ctypes as C
    from dopt_amd import capi
    lib = capi.load()
    r = np.random.default_rng(xs[1] * 7 + k)
    N, Cin, H, W = xs
    ys = (N, k, H, W)
    d = ops.conv_desc(xs, (k, Cin, 3, 3), (1, 1), (1, 1))
    w = ops.tensor((r.standard_normal((k, Cin, 3, 3)) * 0.05).astype(np.float32))
    nbytes = lib.dopt_hip_conv_packed_bytes(C.byref(d), 1)
    assert nbytes > 0
    packed = ops.Tensor([nbytes // 4])
    capi.check(lib.dopt_hip_conv_pack_batch(1, (type(d) * 1)(d), (C.c_int * 1)(1), (C.c_void_p * 1)(w.ptr), (C.c_void_p * 1)(packed.ptr)))
    dy = ops.tensor(r.standard_normal(ys).astype(np.float32))
    x = ops.tensor(r.standard_normal(xs).astype(np.float32))
    dx_want, dw_want = ops.Tensor(xs), ops.Tensor((k, Cin, 3, 3))
    capi.check(lib.dopt_hip_conv_bwd_data_packed(C.byref(d), dy.ptr, packed.ptr, dx_want.ptr))
    capi.check(lib.dopt_hip_conv_bwd_filter(C.byref(d), dy.ptr, x.ptr, dw_want.ptr))
    dx_want, dw_want = dx_want.numpy(), dw_want.numpy()
    dw_scratch = ops.Tensor((k, Cin, 3, 3))
    # closed
    dx, dw = ops.Tensor(xs), ops.Tensor((k, Cin, 3, 3))
    dx.set(np.full(xs, np.nan, np.float32)); dw.set(np.full((k, Cin, 3, 3), np.nan, np.float32))
    capi.check(lib.dopt_hip_conv_pair_probe(1))
    capi.check(lib.dopt_hip_conv_bwd_pair_packed_open(C.byref(d), dy.ptr, packed.ptr, x.ptr, dx.ptr, dw.ptr, None, None))
    n, us, fl, by = C.c_int(), C.c_double(), C.c_double(), C.c_double()
    capi.check(lib.dopt_hip_conv_pair_probe_read(C.byref(n), C.byref(us), C.byref(fl), C.byref(by)))
    capi.check(lib.dopt_hip_conv_pair_probe(0))
    up = lambda v, m: (v + m - 1) // m * m
    # 128-row tiles in both products (wherever 64-row tiles would not pad less) on images of 4 x 4 pixels and more -
    # unless backward-data is a Winograd layer (whole 128-row or 64-row tiles of input channels with a pixel tile of
    # whole 2 x 2 tiles, 64 and more output channels, even sides of at least 4): its filter is packed for that kernel
    # and the two products are two launches
    def winograd_tile(bm, bn):
        padded = bm == 64 and Cin > 64 and (Cin + 63) // 64 * 64 * 5 <= Cin * 6    # 64-row tiles may pad a fifth
        if (Cin % bm and not padded) or bn % W:
            return False
        rows = bn // W
        if rows <= H:
            fits, psz = H % rows == 0 and rows % 2 == 0, (rows + 2) * (W + 2)
        else:
            fits, psz = rows % H == 0, (rows // H) * (H + 2) * (W + 2)
        return fits and psz * 16 <= 16 * 512
    winograd_layer = k % 16 == 0 and k >= 64 and H % 2 == 0 and W % 2 == 0 and H >= 4 and W >= 4
    winograd = winograd_layer and (winograd_tile(128, 128) or winograd_tile(64, 256))
    winograd_open = winograd_layer and winograd_tile(128, 128)     # only the 128-row layers leave the filter gradient open
    one_launch = Cin > 64 and up(Cin, 128) <= up(Cin, 64) and k >= 128 and up(k, 128) <= up(k, 64) and W >= 4 and not winograd
    assert n.value == (1 if one_launch else 0)
    if one_launch:
        assert us.value > 0 and fl.value == 2 * 2.0 * N * H * W * k * Cin * 9
    assert np.array_equal(dx.numpy(), dx_want) and np.array_equal(dw.numpy(), dw_want)
    # open, closed by dopt_hip_split_sum_close
    dx.set(np.full(xs, np.nan, np.float32)); dw.set(np.full((k, Cin, 3, 3), np.nan, np.float32))
    o = capi.SplitSum()
    capi.check(lib.dopt_hip_conv_bwd_pair_packed_open(C.byref(d), dy.ptr, packed.ptr, x.ptr, dx.ptr, dw.ptr, C.byref(o), None))
    assert o.value == dx.ptr
    if xs in ((8, 256, 4, 4), (8, 200, 4, 4)):
        assert o.splits > 1
    if o.splits:
        capi.check(lib.dopt_hip_split_sum_close(C.byref(o)))
    assert np.array_equal(dx.numpy(), dx_want) and np.array_equal(dw.numpy(), dw_want)
    # both left open, both closed by dopt_hip_split_sum_close (the filter gradient first: either order is allowed)
    dx.set(np.full(xs, np.nan, np.float32)); dw.set(np.full((k, Cin, 3, 3), np.nan, np.float32))
    o, ow = capi.SplitSum(), capi.SplitSum()
    capi.check(lib.dopt_hip_conv_bwd_pair_packed_open(C.byref(d), dy.ptr, packed.ptr, x.ptr, dx.ptr, dw.ptr, C.byref(o), C.byref(ow)))
    # (a Winograd backward-data on 128-row tiles and its filter gradient are two launches that leave a split filter
    # gradient open too)
    assert ow.value == dw.ptr and (ow.splits == 0 or ((one_launch or winograd_open) and ow.splits > 1 and ow.lanes in (4, 16)))
    if xs == (16, 200, 8, 8):
        assert ow.splits > 1
    if ow.splits:
        # nothing else may take the workspace while the copies lie in it
        assert lib.dopt_hip_conv_bwd_filter(C.byref(d), dy.ptr, x.ptr, dw_scratch.ptr) != 0
        assert b"was not closed" in lib.dopt_hip_last_error()
        # ... and that refusal drops the library's note of them: the copies themselves are still there
        capi.check(lib.dopt_hip_split_sum_close(C.byref(ow)))
    if o.splits:
        capi.check(lib.dopt_hip_split_sum_close(C.byref(o)))
    assert np.array_equal(dx.numpy(), dx_want) and np.array_equal(dw.numpy(), dw_want)
    # open, closed by the batch-norm gradient one layer down
    inner = H * W
    xin = ops.tensor(r.standard_normal(xs).astype(np.float32))
    yrelu = ops.tensor(np.maximum(r.standard_normal(xs), 0).astype(np.float32))
    sc = ops.tensor(r.uniform(0.5, 1.5, Cin).astype(np.float32))
    g_want, db_want = ops.Tensor([int(np.prod(xs)) + 2 * Cin]), ops.Tensor([Cin])
    capi.check(lib.dopt_hip_bn_grad_fused(N, Cin, inner, ops.tensor(dx_want).ptr, yrelu.ptr, xin.ptr, sc.ptr, g_want.ptr, db_want.ptr))
    g_got, db_got = ops.Tensor([int(np.prod(xs)) + 2 * Cin]), ops.Tensor([Cin])
    dw.set(np.full((k, Cin, 3, 3), np.nan, np.float32))
    o = capi.SplitSum()
    capi.check(lib.dopt_hip_conv_bwd_pair_packed_open(C.byref(d), dy.ptr, packed.ptr, x.ptr, dx.ptr, dw.ptr, C.byref(o), None))
    capi.check(lib.dopt_hip_bn_grad_open(N, Cin, inner, C.byref(o), 1, yrelu.ptr, xin.ptr, sc.ptr, g_got.ptr, db_got.ptr))
    assert np.array_equal(g_got.numpy(), g_want.numpy()) and np.array_equal(db_got.numpy(), db_want.numpy())
    assert np.array_equal(dx.numpy(), dx_want) and np.array_equal(dw.numpy(), dw_want)
    # both open, both closed by ONE batch-norm gradient launch: dx as it is loaded, dw by workgroups that ride along
    g_got.set(np.full(g_got.shape, np.nan, np.float32))
    dx.set(np.full(xs, np.nan, np.float32)); dw.set(np.full((k, Cin, 3, 3), np.nan, np.float32))
    o, ow = capi.SplitSum(), capi.SplitSum()
    capi.check(lib.dopt_hip_conv_bwd_pair_packed_open(C.byref(d), dy.ptr, packed.ptr, x.ptr, dx.ptr, dw.ptr, C.byref(o), C.byref(ow)))
    capi.check(lib.dopt_hip_bn_grad_side(N, Cin, H, W, None, C.byref(o), 1, None, None, yrelu.ptr, xin.ptr, sc.ptr, g_got.ptr,
                                         db_got.ptr, C.byref(ow)))
    assert np.array_equal(g_got.numpy(), g_want.numpy()) and np.array_equal(db_got.numpy(), db_want.numpy())
    assert np.array_equal(dx.numpy(), dx_want) and np.array_equal(dw.numpy(), dw_want)
    # the workspace is free again
    capi.check(lib.dopt_hip_conv_bwd_filter(C.byref(d), dy.ptr, x.ptr, dw_scratch.ptr))
    ops.sync()


def test_batched_products_and_filter_gradients_match_single_calls():
    """dopt_hip_sgemm_batch / dopt_hip_conv_bwd_filter_batch against one dopt_hip_sgemm_t / dopt_hip_conv_bwd_filter per
    job: the jobs that share a launch run the kernel body they would run alone, so every result is identical."""
    lib = capi.load()
    r = np.random.default_rng(70)
    jobs = [(1, 0, 512, 512, 128),    # dense weight gradients: small-output kernel, A stored [K][M]
            (1, 0, 10, 512, 128),
            (1, 0, 512, 512, 128),
            (0, 0, 1, 512, 128),      # bias gradients: short column sums
            (0, 0, 1, 10, 128),
            (1, 0, 37, 1, 100),       # ... of a transposed matrix
            (0, 1, 128, 512, 512),    # small-output kernel, another instance (quads on both operands)
            (0, 0, 70, 33, 50),       # ... and a third (scalar loads)
            (0, 0, 300, 1, 77),       # a row-wise matrix-vector product: runs on its own
            (1, 0, 2048, 2048, 128),  # the LDS-resident panel kernel: on its own
            (0, 0, 16, 4, 1),         # K = 1
            (0, 0, 8, 0, 5)]          # nothing to do
    A, B, want, got = [], [], [], []
    for ta, tb, M, N, K in jobs:
        a = ops.tensor(r.standard_normal((K, M) if ta else (M, K)).astype(np.float32))
        b = ops.tensor(r.standard_normal((N, K) if tb else (K, N)).astype(np.float32))
        w, o = ops.Tensor((M, N)), ops.Tensor((M, N))
        if M * N:
            capi.check(lib.dopt_hip_sgemm_t(ta, tb, M, N, K, a.ptr, b.ptr, w.ptr))
            o.set(np.full((M, N), np.nan, np.float32))
        A.append(a); B.append(b); want.append(w); got.append(o)
    n = len(jobs)
    arr = lambda t, vals: (t * n)(*vals)
    capi.check(lib.dopt_hip_sgemm_batch(n, arr(C.c_int, [j[0] for j in jobs]), arr(C.c_int, [j[1] for j in jobs]),
                                        arr(C.c_size_t, [j[2] for j in jobs]), arr(C.c_size_t, [j[3] for j in jobs]),
                                        arr(C.c_size_t, [j[4] for j in jobs]), arr(C.c_void_p, [t.ptr for t in A]),
                                        arr(C.c_void_p, [t.ptr for t in B]), arr(C.c_void_p, [t.ptr for t in got])))
    for j, w, o in zip(jobs, want, got):
        if j[2] * j[3]:
            assert np.array_equal(o.numpy(), w.numpy()), j
    # filter gradients: three 2x2-image layers in a row share a launch, the 4x4 layer and the narrow one run as ever
    shapes = [((128, 512, 2, 2), 512), ((128, 512, 2, 2), 512), ((128, 256, 2, 2), 512), ((8, 64, 4, 4), 32), ((128, 24, 2, 2), 40),
              ((128, 512, 2, 2), 512)]
    descs, dys, xs, want, got = [], [], [], [], []
    for xshape, k in shapes:
        d = ops.conv_desc(xshape, (k, xshape[1], 3, 3), (1, 1), (1, 1))
        dy = ops.tensor(r.standard_normal((xshape[0], k, xshape[2], xshape[3])).astype(np.float32))
        x = ops.tensor(r.standard_normal(xshape).astype(np.float32))
        w, o = ops.Tensor((k, xshape[1], 3, 3)), ops.Tensor((k, xshape[1], 3, 3))
        capi.check(lib.dopt_hip_conv_bwd_filter(C.byref(d), dy.ptr, x.ptr, w.ptr))
        o.set(np.full(o.shape, np.nan, np.float32))
        descs.append(d); dys.append(dy); xs.append(x); want.append(w); got.append(o)
    n = len(shapes)
    capi.check(lib.dopt_hip_conv_bwd_filter_batch(n, (type(descs[0]) * n)(*descs), (C.c_void_p * n)(*[t.ptr for t in dys]),
                                                  (C.c_void_p * n)(*[t.ptr for t in xs]), (C.c_void_p * n)(*[t.ptr for t in got])))
    for sh, w, o in zip(shapes, want, got):
        assert np.array_equal(o.numpy(), w.numpy()), sh
    ops.sync()


def test_output_only_products_of_a_plan_share_a_launch():
    """The weight and bias gradients of a dense head feed nothing but the plan's outputs: with the rewrites on they are
    one step (`matmul*N`), and so are the filter gradients of consecutive 2x2-image layers; the values are those of the
    plan without rewrites."""
    r = np.random.default_rng(71)
    X = r.standard_normal((128, 3, 8, 8)).astype(np.float32)
    Y = np.eye(10, dtype=np.float32)[r.integers(0, 10, 128)]
    feats, labels = float32([128, 3, 8, 8]), float32([128, 10])
    init = nnet.Init(72)
    body = nnet.vgg(feats, [64, -1, 128, -1, 128, 128], [64], init)     # the last two convolutions see 2x2 images
    preds = nnet.softmax(nnet.dense(body, 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    outs = [loss] + core.grad(loss, net.params)
    plan = core.compile(outs, core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_TIMING)
    fused = plan.execute({feats: X, labels: Y})
    prof = plan.profile()
    # (the product left over is the gradient that flows on into the convolutions: something reads it)
    assert prof["matmul*4"][1] == 1 and prof["matmul"][1] == 1 and "matmul+transpose" not in prof, prof
    assert prof["convolutionFiltersGrad*2"][1] == 1, prof
    plain = core.compile(outs, core.PLAN_VIEWS).execute({feats: X, labels: Y})
    for a, b in zip(plain, fused):
        assert np.array_equal(a, b) or (a.ndim == 1 and np.allclose(a, b, rtol=0, atol=2e-5))


def test_host_arguments_are_consumed_when_the_call_returns():
    """A plan's host arguments (cuda/package.d:367-401 uploads them with a blocking copy) are copied into the plan's
    own page-locked staging memory before the call returns and uploaded beside the kernels still queued, two copies
    taking turns: the caller may overwrite its array at once, and back-to-back executions with different arrays each
    see their own data.  Parameters after six steps equal those of a run that waits after every step."""
    def run(hurry):
        step = configs.softmax_regression(flags=configs.REWRITES)
        feats, labels = step.extra["feats"], step.extra["labels"]
        r = np.random.default_rng(9)
        for k in range(6):
            x = r.random((100, 784)).astype(np.float32)
            y = workloads.one_hot(r.integers(0, 10, 100), 10)
            step.updater.step_async({feats: x, labels: y})
            if hurry:
                x[:] = np.nan            # the call has returned: the arrays are the caller's again
                y[:] = np.nan
            else:
                ops.sync()
        ops.sync()
        return [p.value.copy() for p in step.params]

    a, b = run(True), run(False)
    for u, v in zip(a, b):
        assert np.all(np.isfinite(u)) and np.array_equal(u, v)


def test_weight_decay_terms_square_on_load():
    """`weightDecay * sum(filters * filters)` (nnet/layers/conv.d:117): with the rewrites on the product is never stored
    (`mul+sum`, one pass over the filter); loss and gradients are those of the plan without rewrites, bit for bit.
    Filters of at most 4096 values go into a tiny run instead (here: the first layer's)."""
    r = np.random.default_rng(81)
    X = r.standard_normal((8, 3, 8, 8)).astype(np.float32)
    Y = np.eye(10, dtype=np.float32)[r.integers(0, 10, 8)]
    x, y = core.float32([8, 3, 8, 8]), core.float32([8, 10])
    init = nnet.Init(82)
    h = nnet.relu(nnet.conv2D(nnet.dataSource(x), 32, (3, 3), init, padding=(1, 1), weight_decay=1e-2))
    h = nnet.relu(nnet.conv2D(h, 64, (3, 3), init, padding=(1, 1), weight_decay=1e-2))
    h = nnet.relu(nnet.conv2D(h, 64, (3, 3), init, padding=(1, 1), stride=(2, 2), weight_decay=1e-2))
    top = nnet.softmax(nnet.dense(h, 10, init))
    net = nnet.DAGNetwork([x], [top])
    loss = nnet.crossEntropy(top.trainOutput, y) + net.paramLoss
    outs = [loss] + core.grad(loss, net.params)
    plan = core.compile(outs, core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_TIMING)
    fused = plan.execute({x: X, y: Y})
    prof = plan.profile()
    assert prof["mul+sum"][1] == 2, prof
    plain = core.compile(outs, core.PLAN_VIEWS).execute({x: X, y: Y})
    for a, b in zip(plain, fused):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("M,N,K,ta,tb", [(128, 512, 512, 0, 0),     # the small-output kernel: the epilogue does it
                                          (512, 512, 128, 1, 0),     # a weight gradient: dz stored [K][M]
                                          (10, 512, 128, 1, 0),
                                          (70, 33, 50, 0, 0),        # ragged tiles, scalar loads
                                          (30, 40, 64, 1, 1),
                                          (2048, 2048, 128, 1, 0),   # the LDS-resident panel kernel: separate launches behind it
                                          (1500, 1200, 300, 0, 0),   # the tile engine
                                          (1, 40, 64, 0, 0), (40, 1, 64, 1, 0), (8, 8, 1, 0, 0)])   # vector shapes
def test_products_with_relu_gradient(M, N, K, ta, tb):
    """dopt_hip_sgemm_relu_grad = dopt_hip_sgemm_t then dopt_hip_relu_bwd, bit for bit, whichever kernel runs the product."""
    import ctypes as C
    from dopt_amd import capi
    lib = capi.load()
    r = np.random.default_rng(M * 7 + N + K)
    a = ops.tensor(r.standard_normal((K, M) if ta else (M, K)).astype(np.float32))
    b = ops.tensor(r.standard_normal((N, K) if tb else (K, N)).astype(np.float32))
    x = ops.tensor(r.standard_normal((M, N)).astype(np.float32))
    prod = ops.matmul_t(a, b, bool(ta), bool(tb))
    want = ops.relu_grad(prod, x).numpy()
    got = ops.Tensor((M, N))
    got.set(np.full((M, N), np.nan, np.float32))
    capi.check(lib.dopt_hip_sgemm_relu_grad(ta, tb, M, N, K, a.ptr, b.ptr, x.ptr, got.ptr))
    assert np.array_equal(got.numpy(), want)
    ops.sync()


def test_dense_backward_runs_inside_the_products():
    """With the rewrites on, the relu gradient between two dense layers has no kernel of its own: the product in front of
    it applies the mask.  Values as without the rewrites, bit for bit."""
    r = np.random.default_rng(5)
    X = r.random((64, 96)).astype(np.float32)
    Y = np.zeros((64, 10), np.float32)
    Y[np.arange(64), r.integers(0, 10, 64)] = 1
    feats, labels = float32([64, 96]), float32([64, 10])
    init = nnet.Init(6)
    body = nnet.relu(nnet.dense(nnet.dataSource(feats), 128, init))
    body = nnet.relu(nnet.dense(body, 80, init))
    preds = nnet.softmax(nnet.dense(body, 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    outs = [loss] + core.grad(loss, net.params)
    plan = core.compile(outs, core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_TIMING)
    fused = plan.execute({feats: X, labels: Y})
    prof = plan.profile()
    assert prof["matmul+reluGrad"][1] == 2 and "reluGrad" not in prof, prof
    plain = core.compile(outs, core.PLAN_VIEWS).execute({feats: X, labels: Y})
    for a, b in zip(plain, fused):
        assert np.array_equal(a, b)


def test_dense_backward_keeps_a_product_that_a_batch_norm_gradient_reads():
    """dense -> batch norm -> relu -> dense: the batch-norm gradient applies the relu mask itself and reads the product
    behind the relu gradient, so that product has to stay a plain one - the relu gradient nobody reads any more must not
    pull it into a masked product.  Values as without the rewrites."""
    r = np.random.default_rng(8)
    X = r.standard_normal((64, 48)).astype(np.float32)
    Y = np.zeros((64, 10), np.float32)
    Y[np.arange(64), r.integers(0, 10, 64)] = 1
    feats, labels = float32([64, 48]), float32([64, 10])
    init = nnet.Init(9)
    body = nnet.dense(nnet.dataSource(feats), 32, init)
    as_images = nnet.Layer([body], body.output.reshape([64, 32, 1, 1]), body.trainOutput.reshape([64, 32, 1, 1]), [])
    normed = nnet.relu(nnet.batchNorm(as_images))
    flat = nnet.Layer([normed], normed.output.reshape([64, 32]), normed.trainOutput.reshape([64, 32]), [])
    body = nnet.relu(nnet.dense(flat, 40, init))
    preds = nnet.softmax(nnet.dense(body, 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    outs = [loss] + core.grad(loss, net.params)
    plan = core.compile(outs, core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_TIMING)
    fused = plan.execute({feats: X, labels: Y})
    prof = plan.profile()
    assert prof["matmul+reluGrad"][1] == 1 and "reluGrad" not in prof, prof   # the one between the last two dense layers
    plain = core.compile(outs, core.PLAN_VIEWS).execute({feats: X, labels: Y})
    for a, b in zip(plain, fused):
        if a.ndim <= 1 or a.size == a.shape[0]:
            np.testing.assert_allclose(a, b, rtol=2e-5, atol=1e-6)
        else:
            assert np.array_equal(a, b)


@pytest.mark.parametrize("lanes,splits,n4", [(4, 16, 36864), (16, 37, 1000), (4, 3, 70000)])
@pytest.mark.parametrize("shape,form", [
    ((16, 32, 8, 8), "dy"),            # one workgroup per channel, two quads per lane
    ((128, 16, 16, 16), "dy"),         # eight quads per lane
    ((128, 8, 32, 32), "dy"),          # channels shared by clusters of workgroups
    ((16, 32, 8, 8), "dy_open"),       # dy still in partial copies
    ((16, 32, 8, 8), "pool"),          # dy routed from the gradient of a 2 x 2 max-pool
    ((16, 32, 8, 8), "pool_open"),     # ... which still lies in partial copies
    ((64, 24, 2, 2), "pool_open"),     # 2 x 2 images: a quad is a window
    ((128, 8, 32, 32), "pool_open"),   # in the cluster kernel
    ((16, 12, 8, 12), "pool_open"),    # rows of three quads: pooled by a pass of its own, copies added first
    ((4, 6, 5, 5), "dy"),              # not a register-resident shape: the side sum gets a launch of its own
])
def test_batch_norm_gradient_with_a_sum_riding_along(shape, form, lanes, splits, n4):
    """dopt_hip_bn_grad_side against the separate entry points: the gradient is what dopt_hip_bn_grad_fused /
    dopt_hip_bn_grad_pool give on the finished operands, the side sum what dopt_hip_split_sum_close gives, all to the
    last bit, whichever kernel the shape selects."""
    import ctypes as C
    from dopt_amd import capi
    lib = capi.load()
    r = np.random.default_rng(n4 + shape[1])
    N, Cc, H, W = shape
    x = ops.tensor(r.standard_normal(shape).astype(np.float32))
    y = ops.tensor(np.maximum(r.standard_normal(shape), 0).astype(np.float32))
    sc = ops.tensor(r.uniform(0.5, 1.5, Cc).astype(np.float32))
    total = int(np.prod(shape))

    def open_sum(value_shape, S):
        part = ops.tensor(r.standard_normal((S,) + value_shape).astype(np.float32))
        value = ops.Tensor(value_shape)
        o = capi.SplitSum(part.ptr, S, int(np.prod(value_shape)), value_shape[1], int(np.prod(value_shape[2:])), None, value.ptr, 0)
        return part, value, o

    # the side sum and what closing it gives
    side_part = ops.tensor(r.standard_normal((splits, n4 * 4)).astype(np.float32))
    side_want, side_got = ops.Tensor([n4 * 4]), ops.Tensor([n4 * 4])
    capi.check(lib.dopt_hip_split_sum_close(C.byref(capi.SplitSum(side_part.ptr, splits, n4 * 4, 0, 0, None, side_want.ptr, lanes))))
    side = capi.SplitSum(side_part.ptr, splits, n4 * 4, 0, 0, None, side_got.ptr, lanes)
    side_got.set(np.full(n4 * 4, np.nan, np.float32))

    want, dbw = ops.Tensor([total + 2 * Cc]), ops.Tensor([Cc])
    got, dbg = ops.Tensor([total + 2 * Cc]), ops.Tensor([Cc])
    got.set(np.full(total + 2 * Cc, np.nan, np.float32))
    if form == "dy":
        dy = ops.tensor(r.standard_normal(shape).astype(np.float32))
        capi.check(lib.dopt_hip_bn_grad_fused(N, Cc, H * W, dy.ptr, y.ptr, x.ptr, sc.ptr, want.ptr, dbw.ptr))
        capi.check(lib.dopt_hip_bn_grad_side(N, Cc, H, W, dy.ptr, None, 1, None, None, y.ptr, x.ptr, sc.ptr, got.ptr, dbg.ptr,
                                             C.byref(side)))
    elif form == "dy_open":
        part, dy, o = open_sum(shape, 3)
        capi.check(lib.dopt_hip_split_sum_close(C.byref(o)))
        closed = dy.numpy()
        capi.check(lib.dopt_hip_bn_grad_fused(N, Cc, H * W, dy.ptr, y.ptr, x.ptr, sc.ptr, want.ptr, dbw.ptr))
        dy.set(np.full(shape, np.nan, np.float32))
        capi.check(lib.dopt_hip_bn_grad_side(N, Cc, H, W, None, C.byref(o), 1, None, None, y.ptr, x.ptr, sc.ptr, got.ptr, dbg.ptr,
                                             C.byref(side)))
        assert np.array_equal(dy.numpy(), closed)
    else:
        pshape = (N, Cc, H // 2, W // 2)
        if form == "pool":
            dp = ops.tensor(r.standard_normal(pshape).astype(np.float32))
            o = None
        else:
            part, dp, o = open_sum(pshape, 4)
            capi.check(lib.dopt_hip_split_sum_close(C.byref(o)))
        closed = dp.numpy()
        capi.check(lib.dopt_hip_bn_grad_pool(N, Cc, H, W, dp.ptr, y.ptr, x.ptr, sc.ptr, want.ptr, dbw.ptr))
        if o is not None:
            dp.set(np.full(pshape, np.nan, np.float32))
        capi.check(lib.dopt_hip_bn_grad_side(N, Cc, H, W, None, None, 1, dp.ptr, C.byref(o) if o is not None else None, y.ptr,
                                             x.ptr, sc.ptr, got.ptr, dbg.ptr, C.byref(side)))
        assert np.array_equal(dp.numpy(), closed)
    assert np.array_equal(got.numpy(), want.numpy()) and np.array_equal(dbg.numpy(), dbw.numpy())
    assert np.array_equal(side_got.numpy(), side_want.numpy())
    ops.sync()


@pytest.mark.parametrize("xs,k", [((8, 256, 4, 4), 512),     # split reduction: the result is left open
                                  ((16, 128, 8, 8), 256),
                                  ((2, 64, 32, 32), 64),
                                  ((48, 32, 32, 32), 32),    # channels too large for the resident batch norm: closed first
                                  ((16, 48, 2, 2), 40),      # dense 2x2 route: never open
                                  ((24, 128, 2, 2), 64),     # 2 x 2 images straight from the filter: never open either
                                  ((128, 512, 2, 2), 512)])  # ... at the benchmark shape
def test_open_convolution_results_closed_by_batch_norm(xs, k):
    """The *_open convolutions followed by dopt_hip_bn_train_open / dopt_hip_bn_grad_open /
    dopt_hip_split_sum_close against the closed entry points (checked against the oracle elsewhere):
    the copies are added in the same order, so everything is identical to the last bit."""
    import ctypes as C
    from dopt_amd import capi
    lib = capi.load()
    r = np.random.default_rng(xs[1] + k)
    N, Cin, H, W = xs
    ys = (N, k, H, W)
    d = ops.conv_desc(xs, (k, Cin, 3, 3), (1, 1), (1, 1))
    w = ops.tensor((r.standard_normal((k, Cin, 3, 3)) * 0.05).astype(np.float32))
    packs = []
    for bwd in (0, 1):
        nbytes = lib.dopt_hip_conv_packed_bytes(C.byref(d), bwd)
        assert nbytes > 0
        packs.append(ops.Tensor([nbytes // 4]))
    capi.check(lib.dopt_hip_conv_pack_batch(2, (type(d) * 2)(d, d), (C.c_int * 2)(0, 1), (C.c_void_p * 2)(w.ptr, w.ptr),
                                            (C.c_void_p * 2)(packs[0].ptr, packs[1].ptr)))
    inner = H * W

    # forward: conv + bias -> batch norm + relu
    x = ops.tensor(r.standard_normal(xs).astype(np.float32))
    b = ops.tensor(r.standard_normal(k).astype(np.float32))
    scale, bias = ops.tensor(r.uniform(0.5, 1.5, k).astype(np.float32)), ops.tensor(r.standard_normal(k).astype(np.float32))
    mean, var = ops.tensor(np.zeros(k, np.float32)), ops.tensor(np.ones(k, np.float32))
    conv_want = ops.Tensor(ys)
    capi.check(lib.dopt_hip_conv_fwd_bias_packed(C.byref(d), x.ptr, packs[0].ptr, b.ptr, conv_want.ptr))
    bn_want = ops.bn_train_relu(conv_want, scale, bias, mean, var, 0.9).numpy()
    conv_want = conv_want.numpy()
    for closer in ("bn", "close"):
        conv_got, bn_got = ops.Tensor(ys), ops.Tensor([int(np.prod(ys)) + 2 * k])
        conv_got.set(np.full(ys, np.nan, np.float32))
        o = capi.SplitSum()
        capi.check(lib.dopt_hip_conv_fwd_bias_packed_open(C.byref(d), x.ptr, packs[0].ptr, b.ptr, conv_got.ptr, C.byref(o)))
        assert o.value == conv_got.ptr
        if xs == (8, 256, 4, 4):
            assert o.splits > 1 and o.elems == np.prod(ys) and o.C == k and o.inner == inner
        if xs == (16, 48, 2, 2):
            assert o.splits == 0
        if xs[2:] == (2, 2):
            assert o.splits == 0
        if closer == "close":
            capi.check(lib.dopt_hip_split_sum_close(C.byref(o)))
            o.splits = 0
        capi.check(lib.dopt_hip_bn_train_open(N, k, inner, 0.9, C.byref(o), scale.ptr, bias.ptr, mean.ptr, var.ptr, bn_got.ptr, 1))
        assert np.array_equal(conv_got.numpy(), conv_want)
        assert np.array_equal(bn_got.numpy(), bn_want)

    # backward: conv backward-data -> relu gradient + batch-norm gradient (+ bias gradient)
    dy = ops.tensor(r.standard_normal(ys).astype(np.float32))
    xin = ops.tensor(r.standard_normal(xs).astype(np.float32))         # the batch norm's input one layer down
    yrelu = ops.tensor(np.maximum(r.standard_normal(xs), 0).astype(np.float32))
    sc = ops.tensor(r.uniform(0.5, 1.5, Cin).astype(np.float32))
    dx_want = ops.Tensor(xs)
    capi.check(lib.dopt_hip_conv_bwd_data_packed(C.byref(d), dy.ptr, packs[1].ptr, dx_want.ptr))
    g_want, db_want = ops.Tensor([int(np.prod(xs)) + 2 * Cin]), ops.Tensor([Cin])
    capi.check(lib.dopt_hip_bn_grad_fused(N, Cin, inner, dx_want.ptr, yrelu.ptr, xin.ptr, sc.ptr, g_want.ptr, db_want.ptr))
    dx_want, g_want, db_want = dx_want.numpy(), g_want.numpy(), db_want.numpy()
    for keep in (1, 0):
        dx_got, g_got, db_got = ops.Tensor(xs), ops.Tensor([int(np.prod(xs)) + 2 * Cin]), ops.Tensor([Cin])
        dx_got.set(np.full(xs, 7.0, np.float32))
        o = capi.SplitSum()
        capi.check(lib.dopt_hip_conv_bwd_data_packed_open(C.byref(d), dy.ptr, packs[1].ptr, dx_got.ptr, C.byref(o)))
        was_open = o.splits > 1
        capi.check(lib.dopt_hip_bn_grad_open(N, Cin, inner, C.byref(o), keep, yrelu.ptr, xin.ptr, sc.ptr, g_got.ptr, db_got.ptr))
        assert np.array_equal(g_got.numpy(), g_want)
        assert np.array_equal(db_got.numpy(), db_want)
        if keep or not was_open:
            assert np.array_equal(dx_got.numpy(), dx_want)
        else:   # nobody reads dy: the resident kernel does not write it; the large-channel path closes it first
            got = dx_got.numpy()
            assert np.all(got == 7.0) or np.array_equal(got, dx_want)
            if xs == (8, 256, 4, 4):
                assert np.all(got == 7.0)


def test_an_open_convolution_result_must_be_closed_by_the_next_call():
    """The partial sums of an open result live in the library's workspace; a call that would reuse the workspace
    before they are added up is refused (once), and the library carries on."""
    lib = capi.load()
    r = np.random.default_rng(5)
    xs, ws = (8, 256, 4, 4), (512, 256, 3, 3)
    x = ops.tensor(r.standard_normal(xs).astype(np.float32))
    w = ops.tensor(r.standard_normal(ws).astype(np.float32))
    d = ops.conv_desc(xs, ws, (1, 1), (1, 1))
    nbytes = lib.dopt_hip_conv_packed_bytes(C.byref(d), 0)
    packed = ops.Tensor([nbytes // 4])
    descs = (capi.ConvDesc * 1)(d)
    capi.check(lib.dopt_hip_conv_pack_batch(1, descs, (C.c_int * 1)(0), (C.c_void_p * 1)(w.ptr), (C.c_void_p * 1)(packed.ptr)))
    y = ops.Tensor((8, 512, 4, 4))
    o = capi.SplitSum()
    capi.check(lib.dopt_hip_conv_fwd_bias_packed_open(C.byref(d), x.ptr, packed.ptr, None, y.ptr, C.byref(o)))
    assert o.splits > 1
    with pytest.raises(capi.HipError, match="was not closed"):
        ops.sum(ops.tensor(r.standard_normal((4, 100000)).astype(np.float32)), [1])     # wants the workspace
    # the refusal is reported once; the same convolution, closed properly, gives the plain entry point's result
    capi.check(lib.dopt_hip_conv_fwd_bias_packed_open(C.byref(d), x.ptr, packed.ptr, None, y.ptr, C.byref(o)))
    capi.check(lib.dopt_hip_split_sum_close(C.byref(o)))
    assert np.array_equal(y.numpy(), ops.convolution(x, w, (1, 1), (1, 1)).numpy())


def _small_convnet(seed):
    init = nnet.Init(seed)
    x, y = core.float32([16, 3, 16, 16]), core.float32([16, 10])
    h = nnet.relu(nnet.batchNorm(nnet.conv2D(nnet.dataSource(x), 16, (3, 3), init, padding=(1, 1), weight_decay=1e-3)))
    h = nnet.maxPool(nnet.relu(nnet.batchNorm(nnet.conv2D(h, 32, (3, 3), init, padding=(1, 1)))), (2, 2))
    h = nnet.relu(nnet.batchNorm(nnet.conv2D(h, 32, (3, 3), init, padding=(1, 1), weight_decay=1e-3)))
    top = nnet.softmax(nnet.dense(h, 10, init))
    net = nnet.DAGNetwork([x], [top])
    return x, y, net, nnet.crossEntropy(top.trainOutput, y) + net.paramLoss


@pytest.mark.parametrize("maker", [online.fused_sgd, online.sgd, online.adam])
def test_overlapped_filter_gradients_change_nothing(maker):
    """DOPT_HIP_PLAN_OVERLAP moves the filter gradients (and what only they feed) to a second queue,
    DOPT_HIP_PLAN_OVERLAP_LIGHT the small steps that feed only the outputs (moved up behind their producers):
    the same kernels on the same data, so losses and parameters stay identical bit for bit, step
    after step (every step re-enters buffers the other queue read in the previous one)."""
    r = np.random.default_rng(0)
    xs = r.standard_normal((16, 3, 16, 16)).astype(np.float32)
    ys = np.eye(10, dtype=np.float32)[r.integers(0, 10, 16)]
    base = core.PLAN_VIEWS | core.PLAN_FUSE
    runs = []
    for flags in (base, base | core.PLAN_OVERLAP, base | core.PLAN_OVERLAP_LIGHT, core.PLAN_OVERLAP_LIGHT):
        x, y, net, loss = _small_convnet(4)
        up = maker([loss], net.params, net.paramProj, flags=flags)
        losses = [up({x: xs, y: ys})[0] for _ in range(6)]
        runs.append((losses, [p.value for p in net.params]))
    # the second queue changes nothing (with the rewrites: runs 1, 2 against 0); without the rewrites
    # the bias gradients are summed in another order, so run 3 is compared with a tolerance
    for other in runs[1:3]:
        assert runs[0][0] == other[0]
        for a, b in zip(runs[0][1], other[1]):
            assert np.array_equal(a, b)
    assert np.allclose(runs[0][0], runs[3][0], rtol=1e-4)


def test_second_queue_beside_batch_norms_whose_blocks_share_a_channel():
    """The first two layers of the benchmark network at batch 128 hold 131072 values per channel: their batch norms run
    as four blocks per channel that wait for each other, sized for an otherwise idle device.  With a second queue live
    (both overlap modes) other kernels run beside them; no batch norm is ever moved to that queue, so blocks that wait
    only ever wait for blocks of their own launch, and the steps must stay what they are without the second queue -
    and no launch may report blocks that did not meet."""
    r = np.random.default_rng(5)
    xs = ops.tensor(r.standard_normal((128, 3, 32, 32)).astype(np.float32))
    ys = ops.tensor(np.eye(10, dtype=np.float32)[r.integers(0, 10, 128)])
    base = core.PLAN_VIEWS | core.PLAN_FUSE

    def network(seed):
        init = nnet.Init(seed)
        x, y = core.float32([128, 3, 32, 32]), core.float32([128, 10])
        h = nnet.relu(nnet.batchNorm(nnet.conv2D(nnet.dataSource(x), 64, (3, 3), init, padding=(1, 1))))
        h = nnet.maxPool(nnet.relu(nnet.batchNorm(nnet.conv2D(h, 64, (3, 3), init, padding=(1, 1)))), (2, 2))
        h = nnet.maxPool(nnet.relu(nnet.batchNorm(nnet.conv2D(h, 128, (3, 3), init, padding=(1, 1)))), (2, 2))
        h = nnet.maxPool(h, (2, 2))
        top = nnet.softmax(nnet.dense(nnet.relu(nnet.dense(h, 64, init)), 10, init))
        net = nnet.DAGNetwork([x], [top])
        return x, y, net, nnet.crossEntropy(top.trainOutput, y) + net.paramLoss

    runs = []
    for flags in (base, base | core.PLAN_OVERLAP, base | core.PLAN_OVERLAP_LIGHT):
        x, y, net, loss = network(6)
        up = online.fused_sgd([loss], net.params, net.paramProj, flags=flags)
        losses = [up({x: xs, y: ys})[0] for _ in range(4)]
        ops.sync()                      # raises if a multi-block batch norm gave up waiting
        runs.append((losses, [p.value for p in net.params]))
    for other in runs[1:]:
        assert runs[0][0] == other[0]
        for a, b in zip(runs[0][1], other[1]):
            assert np.array_equal(a, b)


@pytest.mark.parametrize("maker", [online.fused_sgd, online.adam])
def test_recorded_graph_replays_match_direct_execution(maker):
    """DOPT_HIP_PLAN_GRAPH: the first execution with a set of device pointers runs directly, the second
    is recorded, later ones are replays.  Two identically seeded networks take the same steps, one
    through replays and one directly, with the direct one's kernels and host reads interleaved between
    the replays; every loss and, at the end, every parameter must be identical."""
    r = np.random.default_rng(0)
    batches = [(ops.tensor(r.standard_normal((16, 3, 16, 16)).astype(np.float32)),
                ops.tensor(np.eye(10, dtype=np.float32)[r.integers(0, 10, 16)])) for _ in range(2)]
    base = core.PLAN_VIEWS | core.PLAN_FUSE
    xa, ya, neta, lossa = _small_convnet(9)
    xb, yb, netb, lossb = _small_convnet(9)
    direct = maker([lossa], neta.params, neta.paramProj, flags=base)
    replay = maker([lossb], netb.params, netb.paramProj, flags=base | core.PLAN_GRAPH)
    for step in range(8):
        fx, fy = batches[step % 2]        # two bindings: two recordings, each replayed three times
        la = direct({xa: fx, ya: fy})[0]
        lb = replay({xb: fx, yb: fy})[0]
        assert la == lb, step
    for a, b in zip(neta.params, netb.params):
        assert np.array_equal(a.value, b.value)
    assert replay.plan.recordings() == {"recorded": 2, "replays": 4}      # per binding: direct, recorded, 2 replays
    assert direct.plan.recordings() == {"recorded": 0, "replays": 0}
    # host arrays as arguments: every execution uploads anew, so nothing is recorded and nothing breaks
    lb = replay({xb: batches[0][0].numpy(), yb: batches[0][1].numpy()})[0]
    la = direct({xa: batches[0][0].numpy(), ya: batches[0][1].numpy()})[0]
    assert la == lb


def test_recorded_graph_survives_a_workspace_move_and_pool_reuse():
    """A recording holds device addresses.  The library's workspace moves when a later caller needs a larger
    one, and pooled blocks released after a run are handed to new tensors: replays after both events must
    still equal direct execution (the plan records anew instead of launching a stale graph), and tensors
    allocated in between must keep their contents."""
    r = np.random.default_rng(3)
    fx = ops.tensor(r.standard_normal((16, 3, 16, 16)).astype(np.float32))
    fy = ops.tensor(np.eye(10, dtype=np.float32)[r.integers(0, 10, 16)])
    base = core.PLAN_VIEWS | core.PLAN_FUSE
    xa, ya, neta, lossa = _small_convnet(11)
    xb, yb, netb, lossb = _small_convnet(11)
    direct = online.fused_sgd([lossa], neta.params, neta.paramProj, flags=base)
    replay = online.fused_sgd([lossb], netb.params, netb.paramProj, flags=base | core.PLAN_GRAPH)
    for step in range(3):
        assert direct({xa: fx, ya: fy})[0] == replay({xb: fx, yb: fy})[0]
    assert replay.plan.recordings()["recorded"] == 1
    # a filter gradient with a long reduction needs far more workspace than the small network did
    big_x = ops.tensor(r.standard_normal((64, 64, 32, 32)).astype(np.float32))
    big_dy = ops.tensor(r.standard_normal((64, 64, 32, 32)).astype(np.float32))
    ops.conv_bwd_filter(big_dy, big_x, (64, 64, 3, 3), (1, 1), (1, 1))
    ops.sum(ops.tensor(r.standard_normal((4096, 2048)).astype(np.float32)), [0])
    # blocks of every small size class, handed out after the recording and filled with a pattern
    guards = [ops.tensor(np.full(n, 3.25, np.float32)) for n in (64, 256, 1024, 4096, 16384, 65536, 262144, 1 << 20) for _ in range(4)]
    for step in range(3):
        assert direct({xa: fx, ya: fy})[0] == replay({xb: fx, yb: fy})[0]
    for a, b in zip(neta.params, netb.params):
        assert np.array_equal(a.value, b.value)
    for gd in guards:
        assert np.all(gd.numpy() == 3.25)


def test_replayed_multi_block_batch_norm_still_reports_blocks_that_did_not_meet():
    """A plan whose batch norm runs as blocks sharing a channel, replayed as a recorded graph: the error word such a
    kernel raises when its blocks give up (here: the wait bound set to zero by the host, every block still exits) is
    read at the next synchronisation point also when the kernel ran inside a replay, the exchange words are put
    back, and the next replay is correct again."""
    lib = capi.load()
    r = np.random.default_rng(1873)
    shape = (128, 64, 32, 32)                         # 131072 values per channel: four blocks per channel
    X = ops.tensor(r.standard_normal(shape).astype(np.float32))
    ones, zeros = np.ones(64, np.float32), np.zeros(64, np.float32)
    xv = float32(list(shape))
    y, _, _ = core.batchNormTrain(xv, float32([64], ones), float32([64], zeros), float32([64], zeros), float32([64], ones), 0.9)
    plan = core.compile([y], core.PLAN_VIEWS | core.PLAN_GRAPH)
    out = ops.Tensor(shape)
    for _ in range(3):                                # direct, recorded, replayed
        plan.execute({xv: X}, rets=[out])
    ops.sync()
    assert plan.recordings() == {"recorded": 1, "replays": 1}
    want = out.numpy()
    capi.check(lib.dopt_hip_bn_wait_limit(0))
    try:
        # the bound is a kernel argument of the recorded launch: record anew with the bound at zero
        plan2 = core.compile([y], core.PLAN_VIEWS | core.PLAN_GRAPH)
        out2 = ops.Tensor(shape)
        plan2.execute({xv: X}, rets=[out2])           # direct
        with pytest.raises(capi.HipError, match="did not meet"):
            ops.sync()
        plan2.execute({xv: X}, rets=[out2])           # recorded
        with pytest.raises(capi.HipError, match="did not meet"):
            ops.sync()
        plan2.execute({xv: X}, rets=[out2])           # replayed
        assert plan2.recordings() == {"recorded": 1, "replays": 1}
        with pytest.raises(capi.HipError, match="did not meet"):
            ops.sync()
    finally:
        capi.check(lib.dopt_hip_bn_wait_limit(1 << 21))
    ops.sync()
    plan.execute({xv: X}, rets=[out])                 # the first plan's recording: words were put back, result as before
    ops.sync()
    assert plan.recordings()["replays"] == 2
    assert np.array_equal(out.numpy(), want)
    assert_close(want.ravel(), O.bn_train(X.numpy(), ones, zeros, zeros, ones, 0.9)[:want.size], "replayed multi-block batch norm")


def test_graph_flag_leaves_plans_with_caller_registered_kernels_direct():
    """A kernel registered through the C ABI runs host code in execute(); a replay would skip it."""
    lib = core._lib()

    class Kernel(C.Structure):
        _fields_ = [("self", C.c_void_p), ("execute", C.c_void_p), ("destroy", C.c_void_p)]

    EXEC = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.POINTER(C.c_void_p), C.POINTER(C.c_size_t), C.c_void_p,
                       C.c_size_t)
    CTOR = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_int, C.c_void_p, C.POINTER(Kernel))
    calls = []

    def execute(self, nin, inputs, nbytes, out, out_bytes):
        calls.append(1)
        return capi.load().dopt_hip_copy_d2d(out, inputs[0], out_bytes)
    exec_c = EXEC(execute)

    def ctor(graph, op, user, out):
        out[0].self = None
        out[0].execute = C.cast(exec_c, C.c_void_p)
        out[0].destroy = None
        return 0
    ctor_c = CTOR(ctor)
    lib.dopt_hip_deregister_kernel(b"atanh")
    assert lib.dopt_hip_register_kernel(b"atanh", C.cast(ctor_c, C.c_void_p), None) == 0
    try:
        x = core.float32([64])
        plan = core.compile([core.atanh(x) + x], core.PLAN_GRAPH)
        xin, out = ops.tensor(np.arange(64, dtype=np.float32)), ops.Tensor([64])
        for _ in range(4):
            plan.execute({x: xin}, [out])
            assert np.array_equal(out.numpy(), 2 * np.arange(64, dtype=np.float32))
        assert len(calls) == 4
        assert plan.recordings() == {"recorded": 0, "replays": 0}
    finally:
        lib.dopt_hip_deregister_kernel(b"atanh")


def test_graph_flag_leaves_plans_with_random_draws_direct():
    x = core.float32([64], np.ones(64, np.float32))
    y = core.uniformSample([64]) * x
    plan = core.compile([y], core.PLAN_VIEWS | core.PLAN_FUSE | core.PLAN_GRAPH)
    out = ops.Tensor([64])
    draws = []
    for _ in range(4):
        plan.execute(None, [out])
        draws.append(out.numpy().copy())
    assert all(not np.array_equal(draws[0], d) for d in draws[1:])     # a replayed kernel would repeat its draws
