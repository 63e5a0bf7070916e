"""Fixed synthetic workloads shared by the tests and the benchmarks (no reference counterpart:
the reference's examples read datasets; these are the seeded stand-ins of the same shapes)."""
import numpy as np

ADAM16M_TOTAL = 1 << 24


def adam16m_sizes():
    """40 tensor sizes, log-spaced from 4 096 to 2 400 000 elements, totalling 16 777 216.

    The end points are exact; the rounding remainder of the geometric sequence is spread over the
    38 interior tensors in proportion to their size, so most sizes are not multiples of four and
    the multi-tensor kernels' ragged tails are exercised."""
    n, lo, hi = 40, 4096, 2400000
    raw = lo * (hi / lo) ** (np.arange(n) / (n - 1))
    sizes = np.rint(raw).astype(np.int64)
    sizes[0], sizes[-1] = lo, hi
    rest = ADAM16M_TOTAL - int(sizes.sum())
    inner = sizes[1:-1].astype(np.float64)
    add = np.floor(rest * inner / inner.sum()).astype(np.int64)
    sizes[1:-1] += add
    sizes[-2] += rest - int(add.sum())
    assert int(sizes.sum()) == ADAM16M_TOTAL and sizes.min() == lo and (sizes > 0).all()
    return [int(s) for s in sizes]


def adam16m_state(seed=0):
    """Per tensor: w ~ N(0,1), g ~ N(0, 1e-2), m ~ N(0, 1e-2), v = |N(0, 1e-4)| (variances), vhat = v."""
    out = []
    for i, n in enumerate(adam16m_sizes()):
        r = np.random.default_rng([seed, i])
        w = r.standard_normal(n, dtype=np.float32)
        g = r.standard_normal(n, dtype=np.float32) * np.float32(0.1)
        m = r.standard_normal(n, dtype=np.float32) * np.float32(0.1)
        v = np.abs(r.standard_normal(n, dtype=np.float32) * np.float32(0.01))
        out.append({"w": w, "g": g, "m": m, "v": v, "vhat": v.copy()})
    return out


def one_hot(labels, classes=10):
    y = np.zeros((len(labels), classes), np.float32)
    y[np.arange(len(labels)), labels] = 1
    return y
