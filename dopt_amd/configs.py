"""The five benchmark configurations as graphs plus updaters, built with the reference's own constructors
(examples/mnistlogit.d:39-47, nnet/layers/dense.d, nnet/models/vgg.d:54-142, nnet/models/wrn.d:56-219,
online/{sgd,adam,amsgrad}.d).  Inputs are synthetic and seeded; nothing here reads a dataset.

Each builder returns a `Step`: the updater (one call = one training step), the device-resident
arguments of a step, and what a caller needs to check or time it.  Used by bench.py and by the
configuration tests, so both run the same thing.
"""
import numpy as np

from . import core, nnet, online, ops, workloads
from .core import float32

REWRITES = core.PLAN_VIEWS | core.PLAN_FUSE


class Step:
    def __init__(self, name, updater, args, batch, params, loss, extra=None):
        self.name, self.updater, self.args, self.batch = name, updater, args, batch
        self.params, self.loss, self.extra = params, loss, extra or {}

    def run(self, n=1):
        for _ in range(n):
            self.updater.step_async(self.args)

    def loss_value(self):
        return float(self.updater._out_bufs[0].numpy())

    def kernels(self):
        return self.updater.plan.stats()["kernels"]


def _labels(rng, n, classes=10):
    return workloads.one_hot(rng.integers(0, classes, n), classes)


def softmax_regression(flags=0, host_args=False):
    """Config 1: examples/mnistlogit.d:39-47 -- a softmax written out by hand from matmul / maxElement / exp /
    sum / repeat / div on [100, 784] inputs, zero-initialised weights, op-graph SGD with lr 0.1."""
    n = 100
    x = np.random.default_rng(0).random((n, 784)).astype(np.float32)
    y = _labels(np.random.default_rng(1), n)
    feats, labels = float32([n, 784]), float32([n, 10])
    W, b = float32([784, 10]), float32([10])
    linear = core.matmul(feats, W) + core.repeat(b, n)
    numer = core.exp(linear - core.maxElement(linear))
    denom = core.repeat(core.sum(numer, [1]).reshape([n, 1]), [1, 10])
    preds = numer / denom
    loss = nnet.crossEntropy(preds, labels)
    up = online.sgd([loss, preds], [W, b], None, float32([], [0.1]), flags=flags)
    args = {feats: x, labels: y} if host_args else {feats: ops.tensor(x), labels: ops.tensor(y)}
    return Step("config 1: softmax regression [100,784] -> 10, op-graph SGD lr 0.1", up, args, n, [W, b], loss,
                {"feats": feats, "labels": labels, "preds": preds, "x": x, "y": y})


def mlp(fused=True, flags=REWRITES):
    """Config 2: MLP 784-512-512-10, ReLU, softmax cross entropy, batch 256, one ADAM step."""
    n = 256
    x = np.random.default_rng(0).random((n, 784)).astype(np.float32)
    y = _labels(np.random.default_rng(1), n)
    feats, labels = float32([n, 784]), float32([n, 10])
    init = nnet.Init(2)
    body = nnet.relu(nnet.dense(nnet.dataSource(feats), 512, init))
    body = nnet.relu(nnet.dense(body, 512, init))
    preds = nnet.softmax(nnet.dense(body, 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    make = online.fused_adam if fused else online.adam
    up = make([loss, preds.trainOutput], net.params, net.paramProj, flags=flags)
    return Step("config 2: MLP 784-512-512-10 b256, %s ADAM" % ("fused" if fused else "op-graph"), up,
                {feats: ops.tensor(x), labels: ops.tensor(y)}, n, net.params, loss,
                {"feats": feats, "labels": labels, "preds": preds, "net": net, "x": x, "y": y})


class _FusedOnly:
    """Config 3 has no graph: the fused multi-tensor update by itself."""

    def __init__(self, rule):
        st = workloads.adam16m_state(0)
        self.state = st
        self.t = {k: [ops.tensor(s[k]) for s in st] for k in ("w", "g", "m", "v", "vhat")}
        self.opt = ops.FusedOptimizer(self.t["w"], self.t["g"], self.t["m"], self.t["v"],
                                      self.t["vhat"] if rule == "amsgrad" else None)
        self.rule = rule

    def step_async(self, args=None):
        getattr(self.opt, self.rule)(1e-3, 0.9, 0.999, 1e-8)


def fused_update(rule="adam"):
    """Config 3: fused ADAM / AMSGrad over 16 777 216 parameters in 40 tensors."""
    up = _FusedOnly(rule)
    return Step("config 3: fused %s over 16777216 parameters in 40 tensors" % rule, up, None, 0, [], None,
                {"bytes_per_step": workloads.ADAM16M_TOTAL * (28 if rule == "adam" else 36)})


def vgg16(batch=128, fused=True, flags=REWRITES, seed=0):
    """Config 4 (the benchmark): VGG-16 + batch norm on [batch,3,32,32], FC 512-512-10, one SGD(lr 0.01) step."""
    rng = np.random.default_rng(seed)
    feats, labels = float32([batch, 3, 32, 32]), float32([batch, 10])
    init = nnet.Init(seed + 1)
    preds = nnet.softmax(nnet.dense(nnet.vgg16(feats, [512, 512], init), 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    if fused:
        up = online.fused_sgd([loss, preds.trainOutput], net.params, net.paramProj, 0.01, 0.0, flags=flags)
    else:
        up = online.sgd([loss, preds.trainOutput], net.params, net.paramProj, flags=flags)
    x = rng.standard_normal((batch, 3, 32, 32)).astype(np.float32)
    y = _labels(rng, batch)
    return Step("config 4: VGG-16 + batch norm, input [%d,3,32,32], FC 512-512-10, softmax cross-entropy, one "
                "forward + backward + SGD(lr 0.01) step" % batch, up, {feats: ops.tensor(x), labels: ops.tensor(y)},
                batch, net.params, loss, {"feats": feats, "labels": labels, "preds": preds, "net": net, "x": x, "y": y})


def wide_resnet(batch=128, fused=True, flags=REWRITES, depth=28, width=10, seed=0):
    """Config 5: Wide-ResNet-28-10 on [batch,3,32,32], weight decay 1e-4, one ADAM step."""
    rng = np.random.default_rng(seed)
    feats, labels = float32([batch, 3, 32, 32]), float32([batch, 10])
    init = nnet.Init(seed)
    preds = nnet.softmax(nnet.dense(nnet.wideResNet(feats, depth, width, init), 10, init))
    net = nnet.DAGNetwork([feats], [preds])
    loss = nnet.crossEntropy(preds.trainOutput, labels) + net.paramLoss
    make = online.fused_adam if fused else online.adam
    up = make([loss, preds.trainOutput], net.params, net.paramProj, flags=flags)
    x = rng.standard_normal((batch, 3, 32, 32)).astype(np.float32)
    y = _labels(rng, batch)
    return Step("config 5: Wide-ResNet-%d-%d, input [%d,3,32,32], one forward + backward + %s ADAM step" %
                (depth, width, batch, "fused" if fused else "op-graph"), up,
                {feats: ops.tensor(x), labels: ops.tensor(y)}, batch, net.params, loss,
                {"feats": feats, "labels": labels, "preds": preds, "net": net, "x": x, "y": y})


# (C, K, H) of the 13 VGG-16 3x3 pad-1 convolutions on a 32x32 input
VGG_CONVS = [(3, 64, 32), (64, 64, 32), (64, 128, 16), (128, 128, 16), (128, 256, 8), (256, 256, 8), (256, 256, 8),
             (256, 512, 4), (512, 512, 4), (512, 512, 4), (512, 512, 2), (512, 512, 2), (512, 512, 2)]


def conv_flops(n, c, k, h):
    return 2.0 * n * k * c * 9 * h * h


def wrn_conv_flops(batch=128, depth=28, width=10, base=16):
    """2*N*K*C*R*S*P*Q summed over every convolution of the network's forward pass."""
    nblk = (depth - 4) // 6
    total = conv_flops(batch, 3, base, 32)
    cin, h = base, 32
    for mult, s in zip((1, 2, 4), (1, 2, 2)):
        u = base * mult * width
        for i in range(nblk):
            st = s if i == 0 else 1
            ho = h // st
            total += 2.0 * batch * u * cin * 9 * ho * ho          # first 3x3 (strided at a stage entry)
            total += 2.0 * batch * u * u * 9 * ho * ho            # second 3x3
            if cin != u:
                total += 2.0 * batch * u * cin * ho * ho          # 1x1 projection shortcut
            cin, h = u, ho
    return total
