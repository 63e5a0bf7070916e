"""numpy/ctypes binding of the CPU oracle (oracle/dopt_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py, always as the checker and never by the product package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")
F32, I32 = 0, 1


def build(force=False):
    """Compile liboracle.so with the Makefile beside this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "liboracle.so"])
    return _LIB_PATH


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in
                ("N", "C", "H", "W", "K", "R", "S", "padH", "padW", "strideH", "strideW")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
    return _lib


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _sz(seq):
    return (C.c_size_t * max(len(seq), 1))(*[int(s) for s in seq])


def _dt(a):
    if a.dtype == np.float32:
        return F32
    if a.dtype == np.int32:
        return I32
    raise TypeError(a.dtype)


def _chk(rc, what):
    if rc != 0:
        raise RuntimeError("oracle %s failed with code %d" % (what, rc))


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def set_threads(n):
    """Threads for the loops the reference hands to std.parallelism (sum / maxElement over the outer index,
    cpu/math.d:102,179; repeat over its blocks, cpu/basic.d:166).  Results do not depend on it; used by the
    CPU-baseline timing only."""
    lib().oracle_set_threads(int(n))


def get_threads():
    return int(lib().oracle_get_threads())


BINARY = ("add", "sub", "mul", "div", "lt", "lte", "gt", "gte", "eq", "neq", "max", "min", "pow", "atan2")
UNARY = ("neg", "abs", "sgn", "exp", "log", "sqrt", "sin", "cos", "tan", "asin", "acos", "atan",
         "sinh", "cosh", "tanh", "asinh", "acosh", "atanh")


def pointwise(op, a, b=None):
    a = np.ascontiguousarray(a)
    if b is not None:
        b = np.ascontiguousarray(b, dtype=a.dtype)
    out = np.empty_like(a)
    _chk(lib().ref_pointwise(op.encode(), _dt(a), C.c_size_t(a.size), _p(a), _p(b), _p(out)), op)
    return out


def matmul(a, b, f64=False):
    a, b = _f32(a), _f32(b)
    M, K = a.shape
    K2, N = b.shape
    assert K == K2
    out = np.empty((M, N), np.float32)
    fn = lib().f64_matmul if f64 else lib().ref_matmul
    _chk(fn(C.c_size_t(M), C.c_size_t(N), C.c_size_t(K), _p(a), _p(b), _p(out)), "matmul")
    return out


def _reduce(fn, a, axes):
    a = np.ascontiguousarray(a)
    axes = list(range(a.ndim)) if axes is None or len(axes) == 0 else list(axes)
    oshape = [s for i, s in enumerate(a.shape) if i not in axes]
    out = np.empty(oshape, a.dtype)
    _chk(fn(_dt(a), _sz(a.shape), a.ndim, _sz(axes), len(axes), _p(a), _p(out)), "reduce")
    return out


def sum(a, axes=None):  # noqa: A001 - mirrors the reference op name
    return _reduce(lib().ref_sum, a, axes)


def max_element(a, axes=None):
    return _reduce(lib().ref_max_element, a, axes)


def argmin(a, axis):
    a = np.ascontiguousarray(a)
    oshape = list(a.shape)
    oshape[axis] = 1
    out = np.zeros(oshape, np.int32)
    _chk(lib().ref_argmin(_dt(a), _sz(a.shape), a.ndim, C.c_size_t(axis), _p(a), _p(out)), "argmin")
    return out


def slice(a, start, stop):  # noqa: A001
    a = np.ascontiguousarray(a)
    oshape = [e - s for s, e in zip(start, stop)]
    out = np.empty(oshape, a.dtype)
    _chk(lib().ref_slice(a.ndim, _sz(a.shape), _sz(oshape), _sz(start), _p(a), _p(out)), "slice")
    return out


def pad(a, before, after):
    a = np.ascontiguousarray(a)
    oshape = [b + s + e for b, s, e in zip(before, a.shape, after)]
    out = np.full(oshape, 0x55, a.dtype)  # poisoned: the op must write every element
    _chk(lib().ref_pad(a.ndim, _sz(a.shape), _sz(oshape), _sz(before), _p(a), _p(out)), "pad")
    return out


def transpose(a):
    a = np.ascontiguousarray(a)
    out = np.empty((a.shape[1], a.shape[0]), a.dtype)
    _chk(lib().ref_transpose(C.c_size_t(a.shape[0]), C.c_size_t(a.shape[1]), _p(a), _p(out)), "transpose")
    return out


def repeat(a, reps):
    a = np.ascontiguousarray(a)
    oshape = [s * r for s, r in zip(a.shape, reps)]
    out = np.empty(oshape, a.dtype)
    _chk(lib().ref_repeat(a.ndim, _sz(a.shape), _sz(reps), _p(a), _p(out)), "repeat")
    return out


def conv_desc(xshape, wshape, padding=(0, 0), stride=(1, 1)):
    N, Cc, H, W = xshape
    K, C2, R, S = wshape
    assert Cc == C2
    return ConvDesc(N, Cc, H, W, K, R, S, padding[0], padding[1], stride[0], stride[1])


def conv_out_shape(d):
    P = (d.H + 2 * d.padH - d.R) // d.strideH + 1
    Q = (d.W + 2 * d.padW - d.S) // d.strideW + 1
    return (d.N, d.K, P, Q)


def convolution(x, w, padding=(0, 0), stride=(1, 1), f64=True):
    """f64=False is the reference CPU kernel including its bounds quirk."""
    x, w = _f32(x), _f32(w)
    d = conv_desc(x.shape, w.shape, padding, stride)
    y = np.empty(conv_out_shape(d), np.float32)
    fn = lib().f64_conv_fwd if f64 else lib().ref_convolution
    _chk(fn(C.byref(d), _p(x), _p(w), _p(y)), "conv")
    return y


def conv_bwd_data(dy, w, xshape, padding=(0, 0), stride=(1, 1)):
    dy, w = _f32(dy), _f32(w)
    d = conv_desc(xshape, w.shape, padding, stride)
    assert tuple(dy.shape) == conv_out_shape(d)
    dx = np.empty(xshape, np.float32)
    _chk(lib().f64_conv_bwd_data(C.byref(d), _p(dy), _p(w), _p(dx)), "conv_bwd_data")
    return dx


def conv_bwd_filter(dy, x, wshape, padding=(0, 0), stride=(1, 1)):
    dy, x = _f32(dy), _f32(x)
    d = conv_desc(x.shape, wshape, padding, stride)
    assert tuple(dy.shape) == conv_out_shape(d)
    dw = np.empty(wshape, np.float32)
    _chk(lib().f64_conv_bwd_filter(C.byref(d), _p(dy), _p(x), _p(dw)), "conv_bwd_filter")
    return dw


def maxpool(x, dims):
    x = _f32(x)
    N, Cc, H, W = x.shape
    y = np.empty((N, Cc, H // dims[0], W // dims[1]), np.float32)
    _chk(lib().ref_maxpool(*map(C.c_size_t, (N, Cc, H, W, dims[0], dims[1])), _p(x), _p(y)), "maxpool")
    return y


def maxpool_grad(dy, x, dims):
    dy, x = _f32(dy), _f32(x)
    N, Cc, H, W = x.shape
    dx = np.empty_like(x)
    _chk(lib().f64_maxpool_grad(*map(C.c_size_t, (N, Cc, H, W, dims[0], dims[1])), _p(dy), _p(x), _p(dx)),
         "maxpool_grad")
    return dx


def _nci(shape):
    N, Cc = shape[0], shape[1]
    inner = int(np.prod(shape[2:])) if len(shape) > 2 else 1
    return N, Cc, inner


def softmax(x, f64=False):
    x = _f32(x)
    y = np.empty_like(x)
    fn = lib().f64_softmax if f64 else lib().ref_softmax
    _chk(fn(*map(C.c_size_t, _nci(x.shape)), _p(x), _p(y)), "softmax")
    return y


def softmax_grad(dy, y):
    dy, y = _f32(dy), _f32(y)
    dx = np.empty_like(y)
    _chk(lib().f64_softmax_grad(*map(C.c_size_t, _nci(y.shape)), _p(dy), _p(y), _p(dx)), "softmax_grad")
    return dx


def relu(x):
    x = _f32(x)
    y = np.empty_like(x)
    _chk(lib().f64_relu(C.c_size_t(x.size), _p(x), _p(y)), "relu")
    return y


def relu_grad(dy, x):
    dy, x = _f32(dy), _f32(x)
    dx = np.empty_like(x)
    _chk(lib().f64_relu_grad(C.c_size_t(x.size), _p(dy), _p(x), _p(dx)), "relu_grad")
    return dx


def add_bias(x, b):
    x, b = _f32(x), _f32(b)
    y = np.empty_like(x)
    _chk(lib().f64_add_bias(*map(C.c_size_t, _nci(x.shape)), _p(x), _p(b), _p(y)), "add_bias")
    return y


def add_bias_grad(dy):
    dy = _f32(dy)
    db = np.empty((dy.shape[1],), np.float32)
    _chk(lib().f64_add_bias_grad(*map(C.c_size_t, _nci(dy.shape)), _p(dy), _p(db)), "add_bias_grad")
    return db


def bn_train(x, scale, bias, run_mean, run_var, momentum):
    """Returns the packed [y | newRunMean | newRunVar] vector (core/ops/nnet.d:222-225)."""
    x = _f32(x)
    N, Cc, inner = _nci(x.shape)
    packed = np.empty((x.size + 2 * Cc,), np.float32)
    _chk(lib().f64_bn_train(C.c_size_t(N), C.c_size_t(Cc), C.c_size_t(inner), C.c_double(momentum), _p(x),
                            _p(_f32(scale)), _p(_f32(bias)), _p(_f32(run_mean)), _p(_f32(run_var)),
                            _p(packed)), "bn_train")
    return packed


def bn_grad(dy, x, scale):
    """Returns the packed [dx | dscale | dbias] vector (core/ops/nnet.d:232-235)."""
    dy, x = _f32(dy), _f32(x)
    N, Cc, inner = _nci(x.shape)
    packed = np.empty((x.size + 2 * Cc,), np.float32)
    _chk(lib().f64_bn_grad(C.c_size_t(N), C.c_size_t(Cc), C.c_size_t(inner), _p(dy), _p(x), _p(_f32(scale)),
                           _p(packed)), "bn_grad")
    return packed


def bn_infer(x, scale, bias, mean, var):
    x = _f32(x)
    y = np.empty_like(x)
    _chk(lib().f64_bn_infer(*map(C.c_size_t, _nci(x.shape)), _p(x), _p(_f32(scale)), _p(_f32(bias)),
                            _p(_f32(mean)), _p(_f32(var)), _p(y)), "bn_infer")
    return y


def sgd_step(w, g, mom, lr=0.01, mu=0.0, nesterov=False):
    w, g, mom = _f32(w), _f32(g), _f32(mom)
    wo, mo = np.empty_like(w), np.empty_like(w)
    _chk(lib().ref_sgd_step(C.c_size_t(w.size), C.c_float(lr), C.c_float(mu), int(nesterov), _p(w), _p(g),
                            _p(mom), _p(wo), _p(mo)), "sgd")
    return wo, mo


def adam_scalars(alpha, beta1, beta2, b1, b2):
    nb1, nb2, eta = C.c_float(), C.c_float(), C.c_float()
    _chk(lib().ref_adam_scalars(C.c_float(alpha), C.c_float(beta1), C.c_float(beta2), C.c_float(b1),
                                C.c_float(b2), C.byref(nb1), C.byref(nb2), C.byref(eta)), "adam_scalars")
    return nb1.value, nb2.value, eta.value


def adam_step(w, g, m, v, eta, beta1=0.9, beta2=0.999, eps=1e-8):
    w, g, m, v = _f32(w), _f32(g), _f32(m), _f32(v)
    wo, mo, vo = np.empty_like(w), np.empty_like(w), np.empty_like(w)
    _chk(lib().ref_adam_step(C.c_size_t(w.size), C.c_float(eta), C.c_float(beta1), C.c_float(beta2),
                             C.c_float(eps), _p(w), _p(g), _p(m), _p(v), _p(wo), _p(mo), _p(vo)), "adam")
    return wo, mo, vo


def amsgrad_step(w, g, m, v, vhat, eta, beta1=0.9, beta2=0.999, eps=1e-8):
    w, g, m, v, vhat = _f32(w), _f32(g), _f32(m), _f32(v), _f32(vhat)
    wo, mo, vo, vho = (np.empty_like(w) for _ in range(4))
    _chk(lib().ref_amsgrad_step(C.c_size_t(w.size), C.c_float(eta), C.c_float(beta1), C.c_float(beta2),
                                C.c_float(eps), _p(w), _p(g), _p(m), _p(v), _p(vhat), _p(wo), _p(mo), _p(vo),
                                _p(vho)), "amsgrad")
    return wo, mo, vo, vho


def image_transform(batch, jitter_x, jitter_y, geom):
    """ImageTransformer.getBatch on a [N, C, H, W] batch with the random draws given: geom is
    [N, 3] int32 rows of (xOff, yOff, flip X | flip Y << 1)."""
    out = _f32(batch).copy()
    n, c, h, w = out.shape
    g = np.ascontiguousarray(geom, np.int32).reshape(n, 3)
    padded = np.zeros(c * (h + 2 * jitter_y) * (w + 2 * jitter_x), np.float32)
    _chk(lib().ref_image_transform(*map(C.c_size_t, (n, c, h, w, jitter_x, jitter_y)), _p(g), _p(out), _p(padded)),
         "image_transform")
    return out
