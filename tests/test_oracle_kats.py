"""The CPU oracle against every known-answer vector the reference's own unittests hold."""
import numpy as np

import oracle as O


def _arr(vals, shape, dtype):
    return np.array(vals, dtype=dtype).reshape(shape)


def test_slice(kats):
    k = kats["slice"]
    out = O.slice(_arr(k["input"], k["shape"], np.int32), k["start"], k["stop"])
    assert out.ravel().tolist() == k["expected"]


def test_pad(kats):
    k = kats["pad"]
    out = O.pad(_arr(k["input"], k["shape"], np.int32), k["before"], k["after"])
    assert out.shape == (6, 5)
    assert out.ravel().tolist() == k["expected"]


def test_transpose(kats):
    k = kats["transpose"]
    out = O.transpose(_arr(k["input"], k["shape"], np.float32))
    assert out.ravel().tolist() == k["expected"]


def test_repeat(kats):
    for name in ("repeat_1x1", "repeat_2x2"):
        k = kats[name]
        out = O.repeat(_arr(k["input"], k["shape"], np.float32), k["repetitions"])
        assert out.ravel().tolist() == [float(v) for v in k["expected"]]


def test_repeat_by_count_is_matmul_with_ones(kats):
    # core/ops/basic.d:370-381: repeat(n) = ones[n,1] . reshape(x,[1,vol])
    k = kats["repeat_scalar_count"]
    vec = _arr(k["input"], [1, 2], np.float32)
    ones = np.ones((k["repetitions"], 1), np.float32)
    assert O.matmul(ones, vec).ravel().tolist() == k["expected"]


def test_matmul(kats):
    k = kats["matmul"]
    a, b = _arr(k["a"], k["a_shape"], np.float32), _arr(k["b"], k["b_shape"], np.float32)
    assert O.matmul(a, b).ravel().tolist() == k["expected"]
    assert O.matmul(a, b, f64=True).ravel().tolist() == k["expected"]


def test_sum(kats):
    for c in kats["sum"]["cases"]:
        x = _arr(c["input"], c["shape"], np.float32)
        if len(c["shape"]) == 2 and len(c["axes"]) == 1:
            # the op constructor rewrites these to a product with a ones vector
            # (core/ops/math.d:257-279); check both that route and the kernel itself
            ones = np.ones((2, 1), np.float32)
            via_mm = O.matmul(x, ones).ravel() if c["axes"][0] == 1 else O.matmul(ones.T, x).ravel()
            assert via_mm.tolist() == c["expected"]
        assert O.sum(x, c["axes"]).ravel().tolist() == c["expected"]


def test_argmin(kats):
    for c in kats["argmin"]["cases"]:
        out = O.argmin(_arr(c["input"], c["shape"], np.float32), c["axis"])
        assert out.dtype == np.int32
        assert out.ravel().tolist() == c["expected"]


def test_max_element(kats):
    for c in kats["maxElement"]["cases"]:
        out = O.max_element(_arr(c["input"], c["shape"], np.float32), c["axes"])
        assert out.ravel().tolist() == c["expected"]


def test_convolution_pins_filter_flip(kats):
    k = kats["convolution"]
    x = _arr(k["features"], k["features_shape"], np.float32)
    w = _arr(k["filters"], k["filters_shape"], np.float32)
    exp = [float(v) for v in k["expected"]]
    assert O.convolution(x, w, f64=True).ravel().tolist() == exp
    # cross-correlation would give -1 where the reference expects +1
    assert O.convolution(x, w[..., ::-1].copy(), f64=True).ravel().tolist() == [-v if v else 0.0 for v in exp]
    # the CPU kernel tests bounds against the OUTPUT width (4, not 5) so it reads one column less
    ref = O.convolution(x, w, f64=False).ravel().tolist()
    assert ref[:3] == exp[:3] and ref[3] == 0.0


def test_maxpool(kats):
    k = kats["maxpool"]
    out = O.maxpool(_arr(k["input"], k["shape"], np.float32), k["dims"])
    assert out.ravel().tolist() == [np.float32(v) for v in k["expected"]]


def test_softmax(kats):
    k = kats["softmax"]
    x = _arr(k["input"], k["shape"], np.float32)
    for f64 in (False, True):
        out = O.softmax(x, f64=f64).ravel()
        assert np.allclose(out, k["expected"], rtol=k["rel"], atol=k["abs"])
        assert np.allclose(out, k["expected"], rtol=1e-5)


def test_mul_grad_is_r_plus_r():
    # core/grads/package.d:113-129 with mulGrad (core/grads/math.d:79-82):
    # grad = 1*x (from dep 0) + 1*x (from dep 1)
    r = np.float32(37.123456)
    one = np.ones(1, np.float32)
    g0 = O.pointwise("mul", one, np.array([r]))
    g1 = O.pointwise("mul", one, np.array([r]))
    assert O.pointwise("add", g0, g1)[0] == r + r


def test_slice_grad(kats):
    k = kats["slice_grad"]
    a = _arr(k["a"], k["shape"], np.float32)
    b = _arr(k["b"], k["shape"], np.float32)
    # forward c = slice(a*b); grad wrt a = pad(1, before=start, after=shape-stop) * b
    after = [s - e for s, e in zip(k["shape"], k["stop"])]
    padded = O.pad(np.ones((1, 1), np.float32), k["start"], after)
    assert O.pointwise("mul", padded, b).ravel().tolist() == [float(v) for v in k["expected"]]


def test_scalar_plan(kats):
    k = kats["scalar_plan"]
    f = lambda v: np.array([v], np.float32)  # noqa: E731
    assert O.pointwise("add", O.pointwise("mul", f(k["a"]), f(k["b"])), f(k["c"]))[0] == k["expected"]


def test_batchnorm_running_mean_scenario(kats):
    # nnet/layers/batchnorm.d:158-177: the running mean parameter is overwritten each step by
    # the packed newRunMean (projection), x is constant, so mean_t = 0.9*mean_{t-1} + 0.1*mu.
    k = kats["batchnorm_running_mean"]
    x = _arr(k["x"], k["shape"], np.float32)
    C = k["shape"][1]
    gamma, beta = np.ones(C, np.float32), np.zeros(C, np.float32)
    mean, var = np.zeros(C, np.float32), np.ones(C, np.float32)
    for _ in range(k["steps"]):
        packed = O.bn_train(x, gamma, beta, mean, var, float(np.float32(k["momentum"])))
        mean, var = packed[x.size:x.size + C].copy(), packed[x.size + C:].copy()
    assert np.allclose(mean, k["expected_running_mean"], rtol=k["rel"], atol=k["abs"])
    assert np.allclose(mean, k["expected_running_mean"], rtol=1e-5)
