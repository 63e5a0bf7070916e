"""Operator-norm projections (Gouk et al. 2018), restating nnet/source/dopt/nnet/lipschitz.d.

Every function here only composes operations of dopt_amd.core, exactly as the reference composes
its own: the p=2 norms run power iteration as a chain of `matmul` (or `convolution` /
`convolutionTranspose`) nodes started from a fresh `uniformSample`, so on this backend they
exercise the SGEMM, convolution, backward-data and Philox kernels through a compiled plan.
"""
import math

from . import core
from .core import float32, float32Constant, matmul, maxElement, sqrt, transpose, uniformSample


def maxNorm(param, norm, maxval):   # lipschitz.d:162-165
    """param scaled down so that `norm` does not exceed `maxval` (unchanged when it already holds)."""
    return param * (1.0 / core.max(float32([], [1.0]), norm / maxval))


def matrixNorm(param, p, n=2):   # lipschitz.d:42-97
    """The operator norm induced by the vector p-norm, p in {1, 2, inf}.  Weight matrices are stored
    transposed, which is why p=1 sums rows and p=inf sums columns."""
    if param.rank != 2:
        raise ValueError("This function only operates on matrices")
    if p == 1.0:
        return maxElement(core.sum(core.abs(param), [1]))
    if p == 2.0:
        x = uniformSample([param.shape[0], 1]) * 2.0 - 1.0
        weights_t = transpose(param, [1, 0])
        wwt = matmul(param, weights_t)
        for _ in range(n):
            x = matmul(wwt, x)
        v = x / sqrt(core.sum(x * x))
        y = matmul(weights_t, v)
        return sqrt(core.sum(y * y))
    if p == math.inf:
        return maxElement(core.sum(core.abs(param), [0]))
    raise ValueError("Cannot compute matrix norm for p=%s" % p)


def convParamsNorm(param, in_shape, stride, padding, p=2.0, n=2):   # lipschitz.d:113-146
    if p == 2.0:
        x = uniformSample([1, param.shape[1]] + list(in_shape)) * 2.0 - 1.0
        for _ in range(n):
            x = core.convolutionTranspose(core.convolution(x, param, padding, stride), param, padding, stride)
        v = x / sqrt(core.sum(x * x))
        y = core.convolution(v, param, padding, stride)
        return sqrt(core.sum(y * y))
    if p == 1.0 or p == math.inf:
        if param.rank != 2:
            param = param.reshape([param.shape[0], param.volume // param.shape[0]])
        return matrixNorm(param, p)
    raise ValueError("Cannot compute convolution params norm for p=%s" % p)


def projMatrix(maxnorm, p=2.0):   # lipschitz.d:28-38
    def proj(param):
        return maxNorm(param, matrixNorm(param, p), maxnorm)
    return proj


def projConvParams(maxnorm, in_shape, stride, padding, p=2.0):   # lipschitz.d:99-111
    def proj(param):
        return maxNorm(param, convParamsNorm(param, in_shape, stride, padding, p), maxnorm)
    return proj


def maxGainProjection(before, after, maxgain, inner=None):
    """layers/dense.d:113-127, layers/conv.d:129-143, layers/batchnorm.d:97-111: scale the new
    weights by the largest per-example gain ||after|| / ||before|| of the current batch when that
    gain exceeds `maxgain`, then apply the user's own projection, if any."""
    before = before.reshape([before.shape[0], before.volume // before.shape[0]])
    after = after.reshape([after.shape[0], after.volume // after.shape[0]])

    def proj(new_weights):
        before_norms = core.sum(before * before, [1]) + 1e-8
        after_norms = core.sum(after * after, [1]) + 1e-8
        mg = maxElement(sqrt(after_norms / before_norms))
        scaled = new_weights * (1.0 / core.max(float32Constant([], [1.0]), mg / maxgain))
        return scaled if inner is None else inner(scaled)
    return proj


def denseSpectralNorm(weights, num_its=1):   # layers/dense.d:152-169 (the SQUARED norm estimate)
    x = uniformSample([weights.shape[0], 1]) * 2.0 - 1.0
    weights_t = transpose(weights, [1, 0])
    wwt = matmul(weights, weights_t)
    for _ in range(num_its):
        x = matmul(wwt, x)
    v = x / sqrt(core.sum(x * x))
    y = matmul(weights_t, v)
    return core.sum(y * y)


def convSpectralNorm(filters, num_its=1):   # layers/conv.d:174-189: the flattened-filter norm of Yoshida & Miyato
    filters = filters.reshape([filters.shape[0], filters.volume // filters.shape[0]])
    x = uniformSample([filters.shape[1], 1]) * 2.0 - 1.0
    for _ in range(num_its):
        x = matmul(transpose(filters, [1, 0]), matmul(filters, x))
    v = x / sqrt(core.sum(x * x))
    y = matmul(filters, v)
    return core.sum(y * y)
