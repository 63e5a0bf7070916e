"""dopt_hip_tiny_graph: runs of operations on tiny tensors as one launch.  Every node kind against the stand-alone
entry point it stands for, bit for bit (the contract that lets a plan run such a run as one step and still return
what the plan without rewrites returns), and a whole loss tail against the oracle."""
import ctypes as C

import numpy as np
import pytest

import oracle as O
from dopt_amd import capi, ops
from util import assert_close

pytestmark = pytest.mark.gpu

PW, RED, SMAX, SMAXG, REP = range(5)


def _node(kind, dst, a, b=-1, op=0, n=0, a_kind=0, b_kind=0, dims=(0, 0, 0, 0), reps=(0, 0, 0, 0), offs=(0, 0, 0)):
    nd = capi.TinyNode()
    nd.kind, nd.op, nd.dst, nd.a, nd.b, nd.a_kind, nd.b_kind, nd.n = kind, op, dst, a, b, a_kind, b_kind, n
    nd.dst_offset, nd.a_offset, nd.b_offset = offs
    nd.dims = (C.c_int * 4)(*dims)
    nd.reps = (C.c_int * 4)(*reps)
    return nd


def _run(slots, nodes):
    lib = capi.load()
    n = len(nodes)
    capi.check(lib.dopt_hip_tiny_graph(len(slots), (C.c_void_p * len(slots))(*[t.ptr for t in slots]), n,
                                       (capi.TinyNode * n)(*nodes)))


def test_every_pointwise_operation_as_a_node_equals_its_kernel():
    lib = capi.load()
    r = np.random.default_rng(1)
    names = ["add", "sub", "mul", "div", "lt", "lte", "gt", "gte", "eq", "neq", "max", "min", "pow", "atan2", "neg", "abs",
             "sgn", "exp", "log", "sqrt", "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh", "asinh", "acosh",
             "atanh"]
    n = 1000
    a = (r.standard_normal(n) * 2).astype(np.float32)
    b = (r.standard_normal(n) * 2).astype(np.float32)
    a[::50] = b[::50]                                  # equal operands for the comparisons
    a[7], a[8], b[9] = np.nan, np.inf, -np.inf
    ta, tb = ops.tensor(a), ops.tensor(b)
    outs = [ops.Tensor([n]) for _ in names]
    nodes = []
    for k, name in enumerate(names):
        idx = lib.dopt_hip_pointwise_index(name.encode())
        assert idx >= 0
        binary = lib.dopt_hip_pointwise_arity(name.encode()) == 2
        nodes.append(_node(PW, 2 + k, 0, 1 if binary else -1, op=idx, n=n))
    _run([ta, tb] + outs, nodes)
    for name, out in zip(names, outs):
        binary = lib.dopt_hip_pointwise_arity(name.encode()) == 2
        want = ops.pointwise(name, ta, tb if binary else None).numpy()
        assert np.array_equal(out.numpy(), want, equal_nan=True), name
    # relu / reluGrad as nodes against their kernels, a one-element operand, and a column times a row
    relu, rgrad, scal, outer = ops.Tensor([n]), ops.Tensor([n]), ops.Tensor([n]), ops.Tensor([40 * 25])
    one = ops.tensor(np.array([1.25], np.float32))
    _run([ta, tb, relu, rgrad, scal, one, outer],
         [_node(PW, 2, 0, op=lib.dopt_hip_pointwise_index(b"relu"), n=n),
          _node(PW, 3, 0, 1, op=lib.dopt_hip_pointwise_index(b"reluGrad"), n=n),
          _node(PW, 4, 0, 5, op=lib.dopt_hip_pointwise_index(b"mul"), n=n, b_kind=1),
          _node(PW, 6, 0, 1, op=lib.dopt_hip_pointwise_index(b"mul"), n=1000, a_kind=2, b_kind=3, dims=(25, 0, 0, 0))])
    assert np.array_equal(relu.numpy(), ops.relu(ta).numpy(), equal_nan=True)
    assert np.array_equal(rgrad.numpy(), ops.relu_grad(ta, tb).numpy(), equal_nan=True)
    assert np.array_equal(scal.numpy(), a * np.float32(1.25), equal_nan=True)
    want = ops.matmul(ops.tensor(a[:40].reshape(40, 1)), ops.tensor(b[:25].reshape(1, 25))).numpy()
    assert np.array_equal(outer.numpy().reshape(40, 25), want, equal_nan=True)


@pytest.mark.parametrize("shape,axes", [((128, 10), [0, 1]),      # the loss: one contiguous row of 1280 values (quads)
                                        ((1283,), [0]),           # ... of a length that is no multiple of four
                                        ((3, 700), [1]),          # three such rows
                                        ((4095,), [0]),
                                        ((100, 10), [1]),         # short rows: one thread per row
                                        ((12, 30, 7), [1]),       # a strided reduction
                                        ((12, 30, 7), [0, 1]),
                                        ((5, 6, 7, 2), [1, 2]),
                                        ((64,), [0]), ((65,), [0]), ((1,), [0])])
@pytest.mark.parametrize("op", ["sum", "maxElement"])
def test_reductions_as_nodes_equal_dopt_hip_reduce(shape, axes, op):
    r = np.random.default_rng(2)
    x = r.standard_normal(shape).astype(np.float32)
    if op == "maxElement" and x.size > 3:
        x.reshape(-1)[[0, 3]] = np.nan
    tx = ops.tensor(x)
    want = (ops.sum(tx, axes) if op == "sum" else ops.max_element(tx, axes)).numpy()
    outer = int(np.prod(shape[:axes[0]], dtype=np.int64))
    R = int(np.prod([shape[a] for a in axes]))
    inner = int(np.prod(shape[axes[-1] + 1:], dtype=np.int64))
    out = ops.Tensor([max(outer * inner, 1)])
    _run([tx, out], [_node(RED, 1, 0, op=0 if op == "sum" else 1, n=outer * inner, dims=(outer, R, inner, 0))])
    assert np.array_equal(out.numpy().ravel(), want.ravel(), equal_nan=True)


@pytest.mark.parametrize("shape", [(128, 10), (100, 10), (7, 63), (4, 5, 3, 3), (2, 70, 2, 2)])
def test_softmax_nodes_equal_their_kernels(shape):
    r = np.random.default_rng(3)
    x = (r.standard_normal(shape) * 3).astype(np.float32)
    dy = r.standard_normal(shape).astype(np.float32)
    tx, tdy = ops.tensor(x), ops.tensor(dy)
    y = ops.softmax(tx)
    dx = ops.softmax_grad(tdy, y)
    N, Cc = shape[0], shape[1]
    inner = int(np.prod(shape[2:], dtype=np.int64))
    gy, gdx = ops.Tensor(shape), ops.Tensor(shape)
    _run([tx, tdy, gy, gdx], [_node(SMAX, 2, 0, n=x.size, dims=(N, Cc, inner, 0)),
                              _node(SMAXG, 3, 1, 2, n=x.size, dims=(N, Cc, inner, 0))])
    assert np.array_equal(gy.numpy(), y.numpy()) and np.array_equal(gdx.numpy(), dx.numpy())
    assert_close(gy.numpy(), O.softmax(x), "softmax node")


@pytest.mark.parametrize("shape,reps", [((1,), (1000,)), ((3, 4), (2, 5)), ((2, 3, 4, 5), (2, 1, 3, 2)), ((7, 1), (1, 10))])
def test_repeat_node_equals_dopt_hip_repeat(shape, reps):
    r = np.random.default_rng(4)
    x = r.standard_normal(shape).astype(np.float32)
    tx = ops.tensor(x)
    want = ops.repeat(tx, list(reps)).numpy()
    out = ops.Tensor(want.shape)
    lead = 4 - len(shape)
    _run([tx, out], [_node(REP, 1, 0, n=want.size, dims=(1,) * lead + tuple(shape), reps=(1,) * lead + tuple(reps))])
    assert np.array_equal(out.numpy(), want)
    assert np.array_equal(want, np.tile(x, reps))


def test_a_loss_tail_as_one_launch_matches_the_oracle():
    """softmax -> + eps -> log -> * labels -> sum -> * (-1/n), and back: d loss / d logits, as one launch with byte
    offsets into a shared buffer, against the oracle composed operation by operation."""
    lib = capi.load()
    r = np.random.default_rng(5)
    n, c = 128, 10
    logits = (r.standard_normal((n, c)) * 2).astype(np.float32)
    labels = np.eye(c, dtype=np.float32)[r.integers(0, c, n)]
    eps, scale = np.array([1e-6], np.float32), np.array([-1.0 / n], np.float32)
    idx = lambda name: lib.dopt_hip_pointwise_index(name.encode())
    work = ops.Tensor([6 * n * c])                     # y | y + eps | log | labels * log | d/dy | d/dlogits
    loss, total = ops.Tensor([1]), ops.Tensor([1])
    tl, tlab, teps, tsc = ops.tensor(logits), ops.tensor(labels), ops.tensor(eps), ops.tensor(scale)
    B = 4 * n * c
    slots = [tl, tlab, teps, tsc, work, total, loss]
    nodes = [_node(SMAX, 4, 0, n=n * c, dims=(n, c, 1, 0)),
             _node(PW, 4, 4, 2, op=idx("add"), n=n * c, b_kind=1, offs=(B, 0, 0)),
             _node(PW, 4, 4, op=idx("log"), n=n * c, offs=(2 * B, B, 0)),
             _node(PW, 4, 1, 4, op=idx("mul"), n=n * c, offs=(3 * B, 0, 2 * B)),
             _node(RED, 5, 4, op=0, n=1, dims=(1, n * c, 1, 0), offs=(0, 3 * B, 0)),
             _node(PW, 6, 5, 3, op=idx("mul"), n=1),
             # backward: d loss / d y = scale * labels / (y + eps), then through the softmax
             _node(PW, 4, 1, 4, op=idx("div"), n=n * c, offs=(4 * B, 0, B)),
             _node(PW, 4, 4, 3, op=idx("mul"), n=n * c, b_kind=1, offs=(4 * B, 4 * B, 0)),
             _node(SMAXG, 4, 4, 4, n=n * c, dims=(n, c, 1, 0), offs=(5 * B, 4 * B, 0))]
    _run(slots, nodes)
    y = O.softmax(logits)
    want_loss = O.sum(labels * np.log(y + eps[0]), [0, 1]) * scale[0]
    got = work.numpy().reshape(6, n, c)
    assert_close(got[0], y, "softmax")
    assert_close(loss.numpy(), np.asarray(want_loss).reshape(1), "loss")
    dy = (scale[0] * labels / (y + eps[0])).astype(np.float32)
    assert_close(got[5], O.softmax_grad(dy, y), "d loss / d logits")
    # limits are refused, not truncated
    bad = _node(PW, 1, 0, op=idx("neg"), n=5000)
    assert lib.dopt_hip_tiny_graph(2, (C.c_void_p * 2)(tl.ptr, work.ptr), 1, (capi.TinyNode * 1)(bad)) != 0
    assert b"at most" in lib.dopt_hip_last_error()
    ops.sync()
