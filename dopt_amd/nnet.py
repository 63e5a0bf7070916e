"""Graph builders for the layers and models the benchmark configurations use, restating
nnet/source/dopt/nnet/{layers,models,losses,networks,parameters}.d of the reference.

Like dopt_amd.core this is host-side graph construction only (in a deployment it is the
reference's own code): it exists so that the benchmark and the parity tests run the op sequence
the reference would emit for these models.  Parameter initialisation draws from a seeded numpy
generator instead of std.random (the benchmark prescribes its own seeded inputs).
"""
import math

import numpy as np

from . import core
from .core import (addBias, batchNormInference, batchNormTrain, convolution, float32, float32Constant, log, matmul,
                   maxpool, transpose)


class Parameter:   # nnet/parameters.d:14-30
    def __init__(self, symbol, loss=None, projection=None):
        self.symbol, self.loss, self.projection = symbol, loss, projection


class Layer:       # nnet/layers/package.d:30-105
    def __init__(self, deps, output, train_output, params=()):
        self.deps, self.output, self.trainOutput, self.params = list(deps), output, train_output, list(params)


class Init:
    """Seeded stand-in for nnet/parameters.d:33-70 (He / constant initialisers)."""

    def __init__(self, seed=0):
        self.rng = np.random.default_rng(seed)

    def he_gaussian(self, op):   # parameters.d:53-62, fan_in = shape[1] * prod(shape[2:])
        fan_in = int(np.prod(op.shape[1:]))
        op.set_value((self.rng.standard_normal(op.shape) * np.sqrt(2.0 / fan_in)).astype(np.float32))

    @staticmethod
    def constant(op, value):
        op.set_value(np.full(op.shape, value, np.float32))


def dataSource(inputs):   # layers/datasource.d
    return Layer([], inputs, inputs, [])


def _safe_add(a, b):   # layers/dense.d:82-93
    if a is None:
        return b
    return a if b is None else a + b


def dense(inp, num_outputs, init, use_bias=True, weight_decay=0.0, weight_proj=None, bias_proj=None,
          maxgain=math.inf, spectral_decay=0.0):   # layers/dense.d:67-150
    from . import lipschitz
    x, x_tr = inp.output, inp.trainOutput
    x = x.reshape([x.shape[0], x.volume // x.shape[0]])
    x_tr = x_tr.reshape([x_tr.shape[0], x_tr.volume // x_tr.shape[0]])
    weights = float32([num_outputs, x.shape[1]])
    init.he_gaussian(weights)
    weight_loss = None if weight_decay == 0.0 else weight_decay * core.sum(weights * weights)
    weight_loss = _safe_add(weight_loss,
                            None if spectral_decay == 0.0 else spectral_decay * lipschitz.denseSpectralNorm(weights))
    y = matmul(x, transpose(weights, [1, 0]))
    y_tr = matmul(x_tr, transpose(weights, [1, 0]))
    if maxgain != math.inf:
        weight_proj = lipschitz.maxGainProjection(x_tr, y_tr, maxgain, weight_proj)
    params = [Parameter(weights, weight_loss, weight_proj)]
    if use_bias:
        bias = float32([num_outputs])
        y = y + core.repeat(bias, y.shape[0])
        y_tr = y_tr + core.repeat(bias, y_tr.shape[0])
        params.append(Parameter(bias, None, bias_proj))
    return Layer([inp], y, y_tr, params)


def conv2D(inp, out_channels, filter_dims, init, padding=(0, 0), stride=(1, 1), use_bias=True,
           weight_decay=0.0, filter_proj=None, bias_proj=None, maxgain=math.inf,
           spectral_decay=0.0):   # layers/conv.d:66-165
    from . import lipschitz
    x, x_tr = inp.output, inp.trainOutput
    filters = float32([out_channels, x.shape[1]] + list(filter_dims))
    init.he_gaussian(filters)
    filter_loss = None if weight_decay == 0.0 else weight_decay * core.sum(filters * filters)
    filter_loss = _safe_add(filter_loss,
                            None if spectral_decay == 0.0 else spectral_decay * lipschitz.convSpectralNorm(filters))
    y = convolution(x, filters, padding, stride)
    y_tr = convolution(x_tr, filters, padding, stride)
    if maxgain != math.inf:   # measured on the pre-bias response, as the reference does
        filter_proj = lipschitz.maxGainProjection(x_tr, y_tr, maxgain, filter_proj)
    params = [Parameter(filters, filter_loss, filter_proj)]
    if use_bias:
        biases = float32([out_channels])
        y, y_tr = addBias(y, biases), addBias(y_tr, biases)
        params.append(Parameter(biases, None, bias_proj))
    return Layer([inp], y, y_tr, params)


def batchNorm(inp, momentum=0.9, gamma_decay=0.0, gamma_proj=None, beta_proj=None, maxgain=math.inf,
              lipschitz=math.inf):   # layers/batchnorm.d:57-156
    from . import lipschitz as lip
    x, x_tr = inp.output, inp.trainOutput
    c = x.shape[1]
    gamma = float32([1, c, 1, 1], np.ones(c, np.float32))
    beta = float32([c])
    mean = float32([c])
    var = float32([c], np.ones(c, np.float32))
    # the layer holds its momentum as a float and hands it to the op's double attribute
    y_tr, mean_update, var_update = batchNormTrain(x_tr, gamma, beta, mean, var, float(np.float32(momentum)))
    y = batchNormInference(x, gamma, beta, mean, var)
    if maxgain != math.inf:
        # the gain of the scaling alone: the layer's response with zero mean and zero shift
        zeros = float32Constant([c], np.zeros(c, np.float32))
        gamma_proj = lip.maxGainProjection(x_tr, batchNormInference(x_tr, gamma, zeros, zeros, var), maxgain, gamma_proj)
    elif lipschitz != math.inf:
        user_proj = gamma_proj

        def gamma_proj(new_gamma):   # batchnorm.d:113-127: max |gamma / sqrt(var + 1e-6)| held below the bound
            norm = core.maxElement(core.abs(new_gamma / core.sqrt(var_update.reshape(new_gamma.shape) + 1e-6)))
            g = new_gamma * (1.0 / core.max(float32Constant([], [1.0]), norm / lipschitz))
            return g if user_proj is None else user_proj(g)
    gamma_loss = None if gamma_decay == 0.0 else gamma_decay * core.sum(gamma * gamma)
    return Layer([inp], y, y_tr, [Parameter(gamma, gamma_loss, gamma_proj), Parameter(beta, None, beta_proj),
                                  Parameter(mean, None, lambda ignored: mean_update),
                                  Parameter(var, None, lambda ignored: var_update)])


def relu(inp):   # layers/relu.d
    return Layer([inp], core.relu(inp.output), core.relu(inp.trainOutput), [])


def dropout(inp, drop_prob):   # layers/dropout.d:14-33
    x, x_tr = inp.output, inp.trainOutput
    drop_mask = float32(x_tr.shape, np.full(x_tr.volume, drop_prob, np.float32))
    y_tr = core.gt(core.uniformSample(x_tr.shape), drop_mask) * x_tr
    scale = float32(x.shape, np.full(x.volume, 1.0 - drop_prob, np.float32))
    return Layer([inp], x * scale, y_tr, [])


def maxPool(inp, dims):   # layers/maxpool.d
    return Layer([inp], maxpool(inp.output, dims), maxpool(inp.trainOutput, dims), [])


def softmax(inp):   # layers/softmax.d
    return Layer([inp], core.softmax(inp.output), core.softmax(inp.trainOutput), [])


class DAGNetwork:   # nnet/networks.d:20-128
    def __init__(self, inputs, outputs):
        self.inputs, self.outputs = list(inputs), list(outputs)
        order, seen = [], set()

        def visit(layer):
            if id(layer) in seen:
                return
            seen.add(id(layer))
            for d in layer.deps:
                visit(d)
            order.append(layer)
        for o in outputs:
            visit(o)
        self.layers = order
        self.params = [p.symbol for layer in order for p in layer.params]
        self.paramProj = {p.symbol: p.projection for layer in order for p in layer.params if p.projection}
        losses = [p.loss for layer in order for p in layer.params if p.loss is not None]
        self.paramLoss = None
        for term in losses:   # networks.d:48-71: a running sum; a zero scalar variable when there is no term
            self.paramLoss = term if self.paramLoss is None else self.paramLoss + term
        if self.paramLoss is None:
            self.paramLoss = float32([], [0.0])


    def save(self, filename):   # nnet/networks.d:130-143: the parameters' float32 values, back to back, in order
        with open(filename, "wb") as f:
            for p in self.params:
                f.write(np.ascontiguousarray(p.value, "<f4").tobytes())

    def load(self, filename):   # nnet/networks.d:145-160
        with open(filename, "rb") as f:
            for p in self.params:
                raw = f.read(p.volume * 4)
                if len(raw) != p.volume * 4:
                    raise IOError("%s ends before the parameter of shape %s" % (filename, list(p.shape)))
                p.set_value(np.frombuffer(raw, "<f4").reshape(p.shape))


def crossEntropy(hypothesis, ground_truth):   # nnet/losses.d:23-26
    return core.sum(ground_truth * log(hypothesis + 1e-6)) * (-1.0 / hypothesis.shape[0])


def squaredError(hypothesis, ground_truth):   # nnet/losses.d:35-39
    diff = hypothesis - ground_truth
    return core.sum(diff * diff) * (1.0 / hypothesis.shape[0])


VGG16_SIZES = [64, 64, -1, 128, 128, -1, 256, 256, 256, -1, 512, 512, 512, -1, 512, 512, 512, -1]


def vgg(features, extractor_sizes, dense_sizes, init, batchnorm=True):   # nnet/models/vgg.d:54-142
    layers = dataSource(features)
    for s in extractor_sizes:
        if s == -1:
            layers = maxPool(layers, [2, 2])
        else:
            layers = conv2D(layers, s, [3, 3], init, padding=(1, 1))
            if batchnorm:
                layers = batchNorm(layers)
            layers = relu(layers)
    for s in dense_sizes:
        layers = relu(dense(layers, s, init))
    return layers


def vgg16(features, dense_sizes=(4096, 4096), init=None, batchnorm=True):
    return vgg(features, VGG16_SIZES, dense_sizes, init or Init(0), batchnorm)


def _wrn_block(in_layer, u, n, s, init, weight_decay):   # nnet/models/wrn.d:104-200
    res = None
    for _ in range(n):
        res = relu(batchNorm(in_layer))
        res = conv2D(res, u, [3, 3], init, padding=(1, 1), stride=(s, s), use_bias=False, weight_decay=weight_decay)
        res = relu(batchNorm(res))
        res = conv2D(res, u, [3, 3], init, padding=(1, 1), use_bias=False, weight_decay=weight_decay)
        shortcut = in_layer
        if in_layer.output.shape[1] != res.output.shape[1]:
            # 1x1 projection taken from the block INPUT (before its batch norm), no padding
            shortcut = conv2D(in_layer, u, [1, 1], init, stride=(s, s), use_bias=False, weight_decay=weight_decay)
        res = Layer([res, shortcut], res.output + shortcut.output, res.trainOutput + shortcut.trainOutput, [])
        in_layer, s = res, 1
    return res


def meanPool(inp):   # nnet/models/wrn.d:202-219: a row sum (rewritten to a GEMV by `sum`) times 1/(H*W)
    def impl(x):
        n, c, hw = x.shape[0], x.shape[1], x.shape[2] * x.shape[3]
        return core.sum(x.reshape([n * c, hw]), [1]).reshape([n, c]) * (1.0 / hw)
    return Layer([inp], impl(inp.output), impl(inp.trainOutput), [])


def wideResNet(features, depth, width, init=None, weight_decay=0.0001, stride=(1, 2, 2), base=16):
    """nnet/models/wrn.d:56-102 with the default options (no dropout, no norm constraints)."""
    init = init or Init(0)
    n = (depth - 4) // 6
    pred = conv2D(dataSource(features), base, [3, 3], init, padding=(1, 1), use_bias=False, weight_decay=weight_decay)
    for mult, s in zip((1, 2, 4), stride):
        pred = _wrn_block(pred, base * mult * width, n, s, init, weight_decay)
    return meanPool(relu(batchNorm(pred)))
