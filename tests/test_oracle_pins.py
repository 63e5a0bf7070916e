"""Independent pins for the oracle functions the reference's known-answer tests leave open.

Each check is chosen so that a plausible mistake (dropped term, wrong sign or index, transposed
operand, cross-correlation instead of convolution, biased instead of unbiased variance) fails.
Library routines (numpy, scipy, torch CPU in float64) and brute force on tiny inputs are the
independent evidence; nothing here retypes an oracle formula.
"""
import itertools

import numpy as np

import util
import pytest

import oracle as O

rng = np.random.default_rng(1234)


def ulp_diff(a, b):
    a = np.asarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.asarray(b, np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, -(a & 0x7FFFFFFF), a)
    b = np.where(b < 0, -(b & 0x7FFFFFFF), b)
    return np.abs(a - b)


# ---------------------------------------------------------------- pointwise
def test_pointwise_float_exact_ops():
    a = rng.standard_normal(4097).astype(np.float32) * 7
    b = rng.standard_normal(4097).astype(np.float32) * 3
    b[::17] = a[::17]
    exact = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b,
             "lt": (a < b), "lte": (a <= b), "gt": (a > b), "gte": (a >= b), "eq": (a == b),
             "neq": (a != b), "max": np.maximum(a, b), "min": np.minimum(a, b)}
    for op, exp in exact.items():
        out = O.pointwise(op, a, b)
        assert out.dtype == np.float32
        assert np.array_equal(out, exp.astype(np.float32)), op
    un = {"neg": -a, "abs": np.abs(a), "sgn": np.sign(a), "sqrt": np.sqrt(np.abs(a))}
    for op, exp in un.items():
        x = np.abs(a) if op == "sqrt" else a
        assert np.array_equal(O.pointwise(op, x), exp.astype(np.float32)), op


def test_pointwise_float_transcendentals_vs_float64():
    x = (rng.standard_normal(5000) * 4).astype(np.float32)
    p = np.abs(x) + np.float32(1e-3)
    e = (rng.standard_normal(5000)).astype(np.float32)
    checks = [("exp", x, None, np.exp(x.astype(np.float64))),
              ("log", p, None, np.log(p.astype(np.float64))),
              ("pow", p, e, np.power(p.astype(np.float64), e.astype(np.float64))),
              ("sin", x, None, np.sin(x.astype(np.float64))),
              ("tanh", x, None, np.tanh(x.astype(np.float64))),
              ("atan2", x, e, np.arctan2(x.astype(np.float64), e.astype(np.float64)))]
    for op, a, b, exp in checks:
        # exp/log/pow are on the hot path (<= 1 ulp from correctly rounded); the host libm's
        # tanh is a 2-ulp routine
        budget = 1 if op in ("exp", "log", "pow") else 2
        assert ulp_diff(O.pointwise(op, a, b), exp.astype(np.float32)).max() <= budget, op


def test_pointwise_int():
    a = rng.integers(-1000, 1000, 999).astype(np.int32)
    b = rng.integers(1, 50, 999).astype(np.int32) * rng.choice([-1, 1], 999).astype(np.int32)
    assert np.array_equal(O.pointwise("add", a, b), a + b)
    assert np.array_equal(O.pointwise("mul", a, b), a * b)
    # D/C integer division truncates toward zero (numpy floors)
    assert np.array_equal(O.pointwise("div", a, b), np.trunc(a / b).astype(np.int32))
    assert np.array_equal(O.pointwise("lt", a, b), (a < b).astype(np.int32))
    assert np.array_equal(O.pointwise("max", a, b), np.maximum(a, b))
    assert np.array_equal(O.pointwise("neg", a), -a)
    assert np.array_equal(O.pointwise("abs", a), np.abs(a))
    assert np.array_equal(O.pointwise("sgn", a), np.sign(a))
    small = rng.integers(0, 9, 100).astype(np.int32)
    assert np.array_equal(O.pointwise("exp", small), np.exp(small.astype(np.float32)).astype(np.int32))
    assert np.array_equal(O.pointwise("sqrt", np.abs(a)), np.sqrt(np.abs(a).astype(np.float32)).astype(np.int32))
    base = rng.integers(-6, 7, 200).astype(np.int32)
    ex = rng.integers(0, 8, 200).astype(np.int32)
    assert np.array_equal(O.pointwise("pow", base, ex), np.power(base.astype(np.int64), ex).astype(np.int32))
    assert np.array_equal(O.pointwise("add", np.array([2**31 - 1], np.int32), np.array([1], np.int32)),
                          np.array([-2**31], np.int32))  # wraps


# ---------------------------------------------------------------- matmul / reductions / layout
def test_matmul_vs_numpy_float64():
    for M, N, K in [(1, 1, 1), (7, 5, 3), (100, 10, 784), (33, 65, 129), (1, 17, 40), (19, 1, 23)]:
        a = rng.standard_normal((M, K)).astype(np.float32)
        b = rng.standard_normal((K, N)).astype(np.float32)
        exp = a.astype(np.float64) @ b.astype(np.float64)
        assert np.array_equal(O.matmul(a, b, f64=True), exp.astype(np.float32))
        assert np.allclose(O.matmul(a, b), exp, rtol=1e-4, atol=1e-5 * np.sqrt(K))
    # operand order matters: a non-square, non-symmetric case
    a = np.arange(6, dtype=np.float32).reshape(2, 3)
    b = np.arange(12, dtype=np.float32).reshape(3, 4)
    assert np.array_equal(O.matmul(a, b), a @ b)


def test_reductions_bruteforce_all_axis_subsets():
    for shape in [(5,), (3, 4), (2, 3, 4), (2, 3, 2, 3)]:
        xf = rng.integers(-8, 9, shape).astype(np.float32)   # small ints: fp32 sums are exact
        xi = rng.integers(-100, 100, shape).astype(np.int32)
        rank = len(shape)
        for r in range(1, rank + 1):
            for axes in itertools.permutations(range(rank), r):
                for x in (xf, xi):
                    assert np.array_equal(O.sum(x, axes), x.sum(axis=tuple(axes))), (shape, axes)
                    assert np.array_equal(O.max_element(x, axes), x.max(axis=tuple(axes))), (shape, axes)
        for axis in range(rank):
            for x in (xf, xi):
                assert np.array_equal(O.argmin(x, axis), np.argmin(x, axis=axis, keepdims=True).astype(np.int32))


def test_sum_is_a_left_fold_in_fp32():
    # innermost-axis sums fold sequentially in fp32 (cpu/math.d:104-108): 2^24 + 1 + 1 ... stays 2^24
    x = np.array([2.0 ** 24] + [1.0] * 8, np.float32)
    assert O.sum(x)[()] == np.float32(2.0 ** 24)


def test_max_identity_and_argmin_conventions():
    assert O.max_element(np.array([-2**31 + 1, -2**31 + 1], np.int32))[()] == -2**31 + 1
    # all-FLT_MAX lane: strict '<' never fires, the zero-initialised output survives
    assert O.argmin(np.full((1, 4), np.finfo(np.float32).max, np.float32), 1).ravel().tolist() == [0]
    # first minimum wins
    assert O.argmin(np.array([3, 1, 1, 2], np.float32), 0).tolist() == [1]


def test_layout_vs_numpy():
    for shape in [(7,), (4, 6), (3, 4, 5), (2, 3, 4, 5)]:
        x = rng.integers(-1000, 1000, shape).astype(np.int32)
        start = [int(rng.integers(0, s)) for s in shape]
        stop = [int(rng.integers(a + 1, s + 1)) for a, s in zip(start, shape)]
        sl = tuple(slice(a, b) for a, b in zip(start, stop))
        assert np.array_equal(O.slice(x, start, stop), x[sl])
        before = [int(rng.integers(0, 3)) for _ in shape]
        after = [int(rng.integers(0, 3)) for _ in shape]
        assert np.array_equal(O.pad(x, before, after), np.pad(x, list(zip(before, after))))
        reps = [int(rng.integers(1, 4)) for _ in shape]
        assert np.array_equal(O.repeat(x, reps), np.tile(x, reps))
    m = rng.standard_normal((5, 9)).astype(np.float32)
    assert np.array_equal(O.transpose(m), m.T)


# ---------------------------------------------------------------- convolution
def _torch():
    return pytest.importorskip("torch")


CONV_CASES = [  # (N, C, H, W, K, R, S, pad, stride)
    (2, 3, 8, 8, 4, 3, 3, (1, 1), (1, 1)),
    (1, 2, 7, 9, 3, 3, 3, (0, 0), (1, 1)),
    (2, 2, 9, 8, 3, 3, 3, (1, 1), (2, 2)),
    (1, 3, 6, 6, 2, 1, 1, (0, 0), (2, 2)),
    (1, 1, 5, 7, 2, 2, 3, (1, 2), (1, 2)),
]


def test_conv_fwd_vs_scipy_true_convolution():
    from scipy.signal import convolve2d
    x = rng.standard_normal((1, 2, 6, 7)).astype(np.float32)
    w = rng.standard_normal((3, 2, 3, 2)).astype(np.float32)
    y = O.convolution(x, w, f64=True)
    for k in range(3):
        acc = sum(convolve2d(x[0, c].astype(np.float64), w[k, c].astype(np.float64), mode="valid") for c in range(2))
        assert np.allclose(y[0, k], acc, rtol=1e-6, atol=1e-6)


def test_conv_all_three_vs_torch_autograd_float64():
    torch = _torch()
    F = torch.nn.functional
    for (N, C, H, W, K, R, S, pad, st) in CONV_CASES:
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        w = rng.standard_normal((K, C, R, S)).astype(np.float32)
        tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
        tw = torch.tensor(w, dtype=torch.float64, requires_grad=True)
        ty = F.conv2d(tx, tw.flip(2, 3), padding=pad, stride=st)  # true convolution = xcorr with flipped filter
        y = O.convolution(x, w, pad, st, f64=True)
        assert y.shape == tuple(ty.shape)
        assert np.allclose(y, ty.detach().numpy(), rtol=1e-6, atol=1e-6)
        dy = rng.standard_normal(y.shape).astype(np.float32)
        ty.backward(torch.tensor(dy, dtype=torch.float64))
        assert np.allclose(O.conv_bwd_data(dy, w, x.shape, pad, st), tx.grad.numpy(), rtol=1e-6, atol=1e-6)
        assert np.allclose(O.conv_bwd_filter(dy, x, w.shape, pad, st), tw.grad.numpy(), rtol=1e-6, atol=1e-6)


def test_conv_adjoint_identities():
    for (N, C, H, W, K, R, S, pad, st) in CONV_CASES:
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        w = rng.standard_normal((K, C, R, S)).astype(np.float32)
        y = O.convolution(x, w, pad, st)
        dy = rng.standard_normal(y.shape).astype(np.float32)
        lhs = np.vdot(y.astype(np.float64), dy.astype(np.float64))
        assert np.isclose(lhs, np.vdot(x.astype(np.float64), O.conv_bwd_data(dy, w, x.shape, pad, st)), rtol=1e-5)
        assert np.isclose(lhs, np.vdot(w.astype(np.float64), O.conv_bwd_filter(dy, x, w.shape, pad, st)), rtol=1e-5)


def test_cpu_kernel_matches_definition_on_same_shapes():
    # the reference CPU kernel is only valid when output dims == input dims (its bounds quirk)
    x = rng.standard_normal((2, 3, 6, 6)).astype(np.float32)
    w = rng.standard_normal((4, 3, 3, 3)).astype(np.float32)
    assert np.allclose(O.convolution(x, w, (1, 1), (1, 1), f64=False), O.convolution(x, w, (1, 1), (1, 1)),
                       rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------- pooling / softmax / relu / bias
def test_maxpool_and_grad_bruteforce():
    torch = _torch()
    for (H, W, ph, pw) in [(4, 4, 2, 2), (6, 9, 2, 3), (5, 5, 2, 2), (8, 8, 4, 2)]:
        x = rng.standard_normal((2, 3, H, W)).astype(np.float32)
        P, Q = H // ph, W // pw
        blocks = x[:, :, :P * ph, :Q * pw].reshape(2, 3, P, ph, Q, pw)
        assert np.array_equal(O.maxpool(x, (ph, pw)), blocks.max(axis=(3, 5)))
        dy = rng.standard_normal((2, 3, P, Q)).astype(np.float32)
        tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
        torch.nn.functional.max_pool2d(tx, (ph, pw)).backward(torch.tensor(dy, dtype=torch.float64))
        assert np.array_equal(O.maxpool_grad(dy, x, (ph, pw)), tx.grad.numpy().astype(np.float32))


def test_maxpool_grad_tie_goes_to_first_in_row_major_scan():
    x = np.zeros((1, 1, 2, 4), np.float32)
    x[0, 0, :, 2:] = [[1, 5], [5, 5]]
    dx = O.maxpool_grad(np.array([[[[2.0, 3.0]]]], np.float32), x, (2, 2))
    assert dx.ravel().tolist() == [2, 0, 0, 3, 0, 0, 0, 0]


def test_maxpool_grad_follows_the_forward_selection_through_nans():
    """The forward loop keeps acc = (acc < v ? v : acc) from -float.max (cpu/nnet.d:103-113): a NaN never
    replaces acc.  The gradient goes to the element that loop ends up holding; the expected arrays are
    worked out by hand."""
    nan = np.nan
    x = np.array([[[[nan, 1.0, 4.0, nan],
                    [2.0, nan, nan, 4.0]]]], np.float32)
    y = O.maxpool(x, (2, 2))
    assert y.ravel().tolist() == [2.0, 4.0]
    dx = O.maxpool_grad(np.array([[[[7.0, 9.0]]]], np.float32), x, (2, 2))
    # window 0 holds {nan, 1, 2, nan}: 2 at (1, 0); window 1 holds {4, nan, nan, 4}: the first 4 at (0, 2)
    assert dx.ravel().tolist() == [0, 0, 9, 0, 7, 0, 0, 0]
    allnan = np.full((1, 1, 2, 2), nan, np.float32)
    assert O.maxpool(allnan, (2, 2)).ravel().tolist() == [-np.finfo(np.float32).max]
    assert O.maxpool_grad(np.array([[[[5.0]]]], np.float32), allnan, (2, 2)).ravel().tolist() == [5, 0, 0, 0]


def test_softmax_and_grad():
    from scipy.special import softmax as sp_softmax
    x = (rng.standard_normal((4, 7, 3)) * 3).astype(np.float32)
    exp = sp_softmax(x.astype(np.float64), axis=1)
    assert np.allclose(O.softmax(x, f64=True), exp, rtol=1e-6, atol=1e-8)
    assert np.allclose(O.softmax(x), exp, rtol=1e-5, atol=1e-7)
    y = O.softmax(x, f64=True)
    dy = rng.standard_normal(x.shape).astype(np.float32)
    # brute-force Jacobian: J[c,j] = y_c (delta_cj - y_j)
    y64, dy64 = y.astype(np.float64), dy.astype(np.float64)
    jac = np.einsum("nci,cj->ncji", y64, np.eye(7)) - np.einsum("nci,nji->ncji", y64, y64)
    dx = np.einsum("ncji,nci->nji", jac, dy64)
    assert np.allclose(O.softmax_grad(dy, y), dx, rtol=1e-6, atol=1e-7)


def test_relu_and_bias_closed_forms():
    x = rng.standard_normal((3, 5, 4, 2)).astype(np.float32)
    x.flat[::7] = 0.0
    dy = rng.standard_normal(x.shape).astype(np.float32)
    assert np.array_equal(O.relu(x), np.maximum(x, 0))
    assert np.isnan(O.relu(np.array([np.nan], np.float32))[0])
    assert np.array_equal(O.relu_grad(dy, x), np.where(x > 0, dy, 0).astype(np.float32))
    b = rng.standard_normal(5).astype(np.float32)
    assert np.array_equal(O.add_bias(x, b), x + b[None, :, None, None])
    assert np.allclose(O.add_bias_grad(dy), dy.astype(np.float64).sum(axis=(0, 2, 3)), rtol=1e-6)
    x2 = rng.standard_normal((6, 5)).astype(np.float32)
    assert np.array_equal(O.add_bias(x2, b), x2 + b[None, :])


# ---------------------------------------------------------------- batch norm
def test_batchnorm_vs_torch_float64():
    torch = _torch()
    F = torch.nn.functional
    mom = float(np.float32(0.9))
    for shape in [(4, 3, 5, 5), (8, 6), (2, 4, 3, 1)]:
        C = shape[1]
        x = (rng.standard_normal(shape) * 2 + 1).astype(np.float32)
        gamma = rng.standard_normal(C).astype(np.float32)
        beta = rng.standard_normal(C).astype(np.float32)
        rm = rng.standard_normal(C).astype(np.float32)
        rv = (rng.random(C) + 0.5).astype(np.float32)
        dy = rng.standard_normal(shape).astype(np.float32)
        tx = torch.tensor(x, dtype=torch.float64, requires_grad=True)
        tg = torch.tensor(gamma, dtype=torch.float64, requires_grad=True)
        tb = torch.tensor(beta, dtype=torch.float64, requires_grad=True)
        trm, trv = torch.tensor(rm, dtype=torch.float64), torch.tensor(rv, dtype=torch.float64)
        # torch's momentum is the weight of the NEW statistic = 1 - (reference momentum)
        ty = F.batch_norm(tx, trm, trv, tg, tb, training=True, momentum=1.0 - mom, eps=float(np.float32(1e-5)))
        packed = O.bn_train(x, gamma.reshape(1, C, *([1] * (len(shape) - 2))), beta, rm, rv, mom)
        vol = x.size
        assert np.allclose(packed[:vol].reshape(shape), ty.detach().numpy(), rtol=1e-5, atol=1e-6)
        assert np.allclose(packed[vol:vol + C], trm.numpy(), rtol=1e-6, atol=1e-7)
        assert np.allclose(packed[vol + C:], trv.numpy(), rtol=1e-6, atol=1e-7)  # unbiased running variance
        ty.backward(torch.tensor(dy, dtype=torch.float64))
        g = O.bn_grad(dy, x, gamma)
        assert np.allclose(g[:vol].reshape(shape), tx.grad.numpy(), rtol=1e-4, atol=1e-5)
        assert np.allclose(g[vol:vol + C], tg.grad.numpy(), rtol=1e-5, atol=1e-5)
        assert np.allclose(g[vol + C:], tb.grad.numpy(), rtol=1e-5, atol=1e-5)
        tinf = F.batch_norm(torch.tensor(x, dtype=torch.float64), trm, trv, tg, tb, training=False, eps=1e-5)
        # trm/trv were updated in place by the training call above: use them for both sides
        assert np.allclose(O.bn_infer(x, gamma, beta, trm.numpy(), trv.numpy()), tinf.detach().numpy(),
                           rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- optimizers
def _f(v):
    return np.float32(v)


def test_sgd_tree_vs_numpy_float32_nodes():
    n = 1001
    w, g, mom = (rng.standard_normal(n).astype(np.float32) for _ in range(3))
    lr, mu = _f(0.01), _f(0.9)
    nm = mom * mu + lr * g
    wo, mo = O.sgd_step(w, g, mom, lr, mu)
    assert np.array_equal(mo, nm) and np.array_equal(wo, w - nm)
    nm = mom * mu - lr * g
    wo, mo = O.sgd_step(w, g, mom, lr, mu, nesterov=True)
    assert np.array_equal(mo, nm) and np.array_equal(wo, (w + mu * nm) - lr * g)


def test_adam_amsgrad_trees_vs_numpy_float32_nodes():
    n = 1001
    w = rng.standard_normal(n).astype(np.float32)
    g = (rng.standard_normal(n) * 0.1).astype(np.float32)
    m = (rng.standard_normal(n) * 0.1).astype(np.float32)
    v = np.abs(rng.standard_normal(n) * 0.01).astype(np.float32)
    vhat = np.abs(rng.standard_normal(n) * 0.01).astype(np.float32)
    a, b1, b2, eps = _f(1e-3), _f(0.9), _f(0.999), _f(1e-8)
    nb1, nb2, eta = O.adam_scalars(a, b1, b2, 1.0, 1.0)
    assert _f(nb1) == b1 and _f(nb2) == b2
    assert _f(eta) == (a * np.sqrt(_f(1) - b2)) / (_f(1) - b1)
    nm = b1 * m + (_f(1) - b1) * g
    nv = b2 * v + ((_f(1) - b2) * g) * g
    nw = w - _f(eta) * (nm / (np.sqrt(nv) + eps))
    wo, mo, vo = O.adam_step(w, g, m, v, eta, b1, b2, eps)
    assert np.array_equal(mo, nm) and np.array_equal(vo, nv) and np.array_equal(wo, nw)
    wo, mo, vo, vho = O.amsgrad_step(w, g, m, v, vhat, eta, b1, b2, eps)
    assert np.array_equal(wo, nw) and np.array_equal(vho, np.maximum(vhat, v))  # OLD v, and w uses v'


@pytest.mark.parametrize("which", ["sgd", "adam", "amsgrad"])
def test_fit_line_scenario(which):
    # online/{sgd,adam,amsgrad}.d unittests: fit y = 3x + 2, one sample per step, expect m->3, c->2
    r = np.random.default_rng(7)
    xs = r.uniform(-10, 10, 100).astype(np.float32)
    ys = _f(3) * xs + _f(2)
    p = np.zeros(2, np.float32)                       # [m, c]
    st = [np.zeros(2, np.float32) for _ in range(3)]  # mom | m, v, vhat
    b1 = b2 = 1.0
    steps = 300 if which == "sgd" else 3000
    for i in range(steps):
        x, y = xs[i % 100], ys[i % 100]
        d = (p[0] * x + p[1]) - y
        g = np.array([(d + d) * x, d + d], np.float32)   # grads of (yhat-y)^2 through mulGrad/addGrad
        if which == "sgd":
            p, st[0] = O.sgd_step(p, g, st[0], 0.001, 0.9)
        else:
            b1, b2, eta = O.adam_scalars(0.1, 0.9, 0.999, b1, b2)
            if which == "adam":
                p, st[0], st[1] = O.adam_step(p, g, st[0], st[1], eta)
            else:
                p, st[0], st[1], st[2] = O.amsgrad_step(p, g, st[0], st[1], st[2], eta)
    assert abs(p[0] - 3) < 0.05 and abs(p[1] - 2) < 0.3, p


# ----------------------------------------------------------------------------- Philox (checker of `uniform`)
def test_numpy_philox_matches_published_vectors():
    # Random123 kat_vectors, philox4x32 with 10 rounds
    z = util.philox4x32_10(np.zeros((1, 4), np.uint32), [0, 0])[0]
    assert [hex(v) for v in z] == ["0x6627e8d5", "0xe169c58d", "0xbc57ac4c", "0x9b00dbd8"]
    f = util.philox4x32_10(np.full((1, 4), 0xFFFFFFFF, np.uint32), [0xFFFFFFFF, 0xFFFFFFFF])[0]
    assert [hex(v) for v in f] == ["0x408f276d", "0x41c83b0e", "0xa20bc7c6", "0x6d5451fd"]
    p = util.philox4x32_10(np.array([[0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344]], np.uint32), [0xA4093822, 0x299F31D0])[0]
    assert [hex(v) for v in p] == ["0xd16cfe09", "0x94fdcceb", "0x5001e420", "0x24126ea1"]
