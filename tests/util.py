import numpy as np


def ulp_diff(a, b):
    """Distance in units in the last place between two float32 arrays (NaN pairs count as 0)."""
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    both_nan = np.isnan(a) & np.isnan(b)
    ai = a.view(np.int32).astype(np.int64)
    bi = b.view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, -(ai & 0x7FFFFFFF), ai)
    bi = np.where(bi < 0, -(bi & 0x7FFFFFFF), bi)
    d = np.abs(ai - bi)
    return np.where(both_nan, 0, d)


# north_star tolerances
GEMM_RTOL, GEMM_ATOL = 1e-4, 1e-5


def assert_close(got, want, what="", rtol=GEMM_RTOL, atol=GEMM_ATOL, scale=None):
    """|got - want| <= atol*scale + rtol*|want|.  `scale` rescales atol for reductions whose terms
    are far from O(1) (a length-n dot product of N(0,1) terms has magnitude sqrt(n))."""
    got = np.asarray(got, np.float64)
    want = np.asarray(want, np.float64)
    tol = atol * (scale if scale else 1.0) + rtol * np.abs(want)
    bad = np.abs(got - want) > tol
    if bad.any():
        i = np.argmax(np.abs(got - want) - tol)
        raise AssertionError("%s: %d/%d outside tolerance; worst at %d: got %r want %r" %
                             (what, bad.sum(), bad.size, i, got.ravel()[i], want.ravel()[i]))


# Rows of (case, quantity, max |err|, max |err| / (atol + rtol |want|), max |want|) collected by the
# configuration tests; conftest.py writes them to parity_errors.txt at the end of a session (see there).
ERROR_ROWS = []


def err_ratio(got, want, what=None, case=None, rtol=GEMM_RTOL, atol=GEMM_ATOL):
    """max |got - want| / (atol + rtol |want|): at most 1 exactly when assert_close(got, want) with the same
    unscaled tolerance passes.  Recorded under (case, what) when both are given."""
    got = np.asarray(got, np.float64).ravel()
    want = np.asarray(want, np.float64).ravel()
    assert got.shape == want.shape, (what, got.shape, want.shape)
    err = np.abs(got - want)
    ratio = float((err / (atol + rtol * np.abs(want))).max()) if err.size else 0.0
    if not np.isfinite(got).all():
        ratio = float("inf")
    if what is not None:
        ERROR_ROWS.append((case or "", what, float(err.max()) if err.size else 0.0, ratio,
                           float(np.abs(want).max()) if want.size else 0.0))
    return ratio


M0, M1, W0, W1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85


def philox4x32_10(ctr, key):
    """numpy restatement of the published algorithm; ctr is [n, 4] uint32, key [2]."""
    c = [ctr[:, i].astype(np.uint64) for i in range(4)]
    k0, k1 = np.uint64(key[0]), np.uint64(key[1])
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0, p1 = np.uint64(M0) * c[0], np.uint64(M1) * c[2]
        hi0, lo0, hi1, lo1 = p0 >> np.uint64(32), p0 & mask, p1 >> np.uint64(32), p1 & mask
        c = [hi1 ^ c[1] ^ k0, lo1, hi0 ^ c[3] ^ k1, lo0]
        k0, k1 = (k0 + np.uint64(W0)) & mask, (k1 + np.uint64(W1)) & mask
    return np.stack(c, axis=1).astype(np.uint32)
