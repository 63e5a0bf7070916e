"""Parity of every kernel entry point of libdopthip.so (through the C ABI) against the CPU oracle.

Tolerances are the ones the project states: bit-exact for integer, index and layout work and
for single-rounding fp32 arithmetic; <= 2 ulp for fp32 transcendentals; rtol 1e-4 / atol 1e-5
for GEMM, convolution and reductions.  Where a test sums n products of N(0,1) numbers the sum itself
has magnitude sqrt(n) and atol is scaled by that; the same kernel is then run again on operands scaled
as the configurations scale them (He-scaled weights, gradients that carry the 1/batch of a mean loss),
where results are O(1) or smaller, and must meet the stated tolerance with no rescaling.
"""
import numpy as np
import pytest

import oracle as O
from util import assert_close, ulp_diff

pytestmark = pytest.mark.gpu

from dopt_amd import ops
T = ops.tensor


def rng(seed):
    return np.random.default_rng(seed)


# ----------------------------------------------------------------------------- runtime
def test_buffer_roundtrip_zero_fill_and_pool_reuse():
    from dopt_amd import capi
    import ctypes as C
    lib = capi.load()
    a = rng(0).standard_normal(100003).astype(np.float32)
    t = T(a)
    assert np.array_equal(t.numpy(), a)
    z = ops.Tensor((4097,), np.int32)
    assert not z.numpy().any()                      # CUDABuffer.create zero-fills
    with pytest.raises(capi.HipError):
        z.set(np.zeros(5, np.int32))                # "input buffer is the wrong length."
    allocs0 = C.c_size_t()
    lib.dopt_hip_pool_stats(None, None, C.byref(allocs0))
    ptr = z.ptr
    z.free()
    z2 = ops.Tensor((4097,), np.int32)
    allocs1 = C.c_size_t()
    lib.dopt_hip_pool_stats(None, None, C.byref(allocs1))
    assert z2.ptr == ptr and allocs1.value == allocs0.value   # served from the pool
    assert not z2.numpy().any()


# ----------------------------------------------------------------------------- pointwise
@pytest.mark.parametrize("n", [1, 3, 4, 1023, 4096, 100003, 1 << 20])
def test_pointwise_f32_exact(n):
    r = rng(n)
    a = (r.standard_normal(n) * 5).astype(np.float32)
    b = (r.standard_normal(n) * 3).astype(np.float32)
    b[::13] = a[::13]
    ta, tb = T(a), T(b)
    for op in ["add", "sub", "mul", "div", "lt", "lte", "gt", "gte", "eq", "neq", "max", "min"]:
        assert np.array_equal(ops.pointwise(op, ta, tb).numpy(), O.pointwise(op, a, b)), op
    for op in ["neg", "abs", "sgn"]:
        assert np.array_equal(ops.pointwise(op, ta).numpy(), O.pointwise(op, a)), op
    pa = np.abs(a)
    assert np.array_equal(ops.pointwise("sqrt", T(pa)).numpy(), O.pointwise("sqrt", pa))


def test_pointwise_f32_transcendentals():
    r = rng(5)
    n = 200001
    x = (r.standard_normal(n) * 4).astype(np.float32)
    p = (np.abs(x) + 1e-3).astype(np.float32)
    e = r.standard_normal(n).astype(np.float32)
    small = (r.uniform(-0.99, 0.99, n)).astype(np.float32)
    cases = [("exp", x, None), ("log", p, None), ("pow", p, e), ("sin", x, None), ("cos", x, None),
             ("tanh", x, None), ("atan", x, None), ("atan2", x, e), ("asin", small, None), ("sinh", x, None)]
    for op, a, b in cases:
        got = ops.pointwise(op, T(a), T(b) if b is not None else None).numpy()
        want = O.pointwise(op, a, b)
        # exp/log/pow are what the reference's device backend registers (cuda/math.d:117-127): <= 2 ulp.
        # The remaining functions reach the reference only through its host fallback; the device
        # math library documents up to 3-4 ulp for some of them.
        budget = 2 if op in ("exp", "log", "pow") else 4
        assert ulp_diff(got, want).max() <= budget, (op, ulp_diff(got, want).max())


def test_pointwise_unaligned_views_take_the_scalar_path():
    a = rng(1).standard_normal(1001).astype(np.float32)
    b = rng(2).standard_normal(1001).astype(np.float32)
    ta, tb = T(a), T(b)
    va, vb = ta.view(1, (1000,)), tb.view(1, (1000,))
    assert np.array_equal(ops.pointwise("mul", va, vb).numpy(), a[1:] * b[1:])


def test_pointwise_i32():
    r = rng(3)
    n = 10007
    a = r.integers(-1000, 1000, n).astype(np.int32)
    b = (r.integers(1, 50, n) * r.choice([-1, 1], n)).astype(np.int32)
    ta, tb = T(a), T(b)
    for op in ["add", "sub", "mul", "div", "lt", "lte", "gt", "gte", "eq", "neq", "max", "min"]:
        got = ops.pointwise(op, ta, tb)
        assert got.dtype == np.int32
        assert np.array_equal(got.numpy(), O.pointwise(op, a, b)), op
    for op in ["neg", "abs", "sgn"]:
        assert np.array_equal(ops.pointwise(op, ta).numpy(), O.pointwise(op, a)), op
    base, ex = r.integers(-6, 7, n).astype(np.int32), r.integers(0, 8, n).astype(np.int32)
    assert np.array_equal(ops.pointwise("pow", T(base), T(ex)).numpy(), O.pointwise("pow", base, ex))
    pos = np.abs(a)
    assert np.array_equal(ops.pointwise("sqrt", T(pos)).numpy(), O.pointwise("sqrt", pos))
    big = np.array([2**31 - 1, -2**31], np.int32)
    one = np.array([1, -1], np.int32)
    assert np.array_equal(ops.pointwise("add", T(big), T(one)).numpy(), O.pointwise("add", big, one))


def test_pointwise_rejects_bad_arity_and_names():
    from dopt_amd import capi
    a = T(np.ones(4, np.float32))
    with pytest.raises(capi.HipError):
        ops.pointwise("add", a)
    with pytest.raises(capi.HipError):
        ops.pointwise("bogus", a, a)


# ----------------------------------------------------------------------------- reductions
@pytest.mark.parametrize("shape,axes", [
    ((128, 10), None), ((100, 10), None), ((7,), None), ((3, 4, 5), (1,)), ((3, 4, 5), (0, 2)),
    ((2, 3, 4, 5), (1, 2)), ((2, 3, 4, 5), (3,)), ((2, 3, 4, 5), (0,)), ((640, 640, 3, 3), None),
    ((5, 70000), (1,)), ((2048, 33), (1,)), ((4, 6), (0,)),
    # everything but a run of axes in the middle (a per-channel statistic): the one-launch sliced kernel
    ((128, 64, 32, 32), (0, 2, 3)), ((16, 8, 16, 32), (0, 2, 3)), ((3, 5, 7, 300), (0, 3)), ((70, 3, 2, 258), (0, 3)),
    ((2, 3, 100000), None),                       # one row split over many blocks, finished by the last of them
    ((3, 2 * 4096 * 5 + 8), (1,)),                # the same for several rows
])
def test_sum_and_max(shape, axes):
    r = rng(11)
    x = r.standard_normal(shape).astype(np.float32)
    red = int(np.prod([shape[a] for a in (axes or range(len(shape)))]))
    got = ops.sum(T(x), axes).numpy()
    want64 = x.astype(np.float64).sum(axis=tuple(axes) if axes else None)
    assert got.shape == np.asarray(want64).shape
    assert_close(got, want64, "sum", scale=np.sqrt(red))
    xm = (x * np.float32(1.0 / np.sqrt(red))).astype(np.float32)      # sums of O(1): stated tolerance as it stands
    assert_close(ops.sum(T(xm), axes).numpy(), xm.astype(np.float64).sum(axis=tuple(axes) if axes else None), "sum, O(1)")
    if red <= 4096:  # the reference's own fp32 left-fold is itself within tolerance of the device result
        assert_close(got, O.sum(x, axes), "sum vs reference order", scale=np.sqrt(red))
    assert np.array_equal(ops.max_element(T(x), axes).numpy(), O.max_element(x, axes))
    xi = r.integers(-1000, 1000, shape).astype(np.int32)
    assert np.array_equal(ops.sum(T(xi), axes).numpy(), O.sum(xi, axes))
    assert np.array_equal(ops.max_element(T(xi), axes).numpy(), O.max_element(xi, axes))


@pytest.mark.parametrize("shape,axes", [
    ((640, 640, 3, 3), None), ((320, 160, 1, 1), None), ((7,), None), ((3, 4, 5), (1,)), ((3, 4, 5), (0, 2)),
    ((5, 70001), (1,)), ((2048, 33), (1,)), ((4, 6), (0,)), ((16, 8, 16, 32), (0, 2, 3)), ((2, 3, 100000), None),
    ((0, 4), (0,)),
])
def test_sum_of_squares_is_the_sum_of_the_stored_product(shape, axes):
    """dopt_hip_reduce_squares against mul followed by sum, bit for bit (one launch less and the product never stored),
    and against float64 within the stated tolerance; also from a buffer off the 16-byte grid."""
    r = rng(13)
    x = r.standard_normal(shape).astype(np.float32)
    got = ops.sum_of_squares(T(x), axes).numpy()
    two = ops.sum(ops.pointwise("mul", T(x), T(x)), axes).numpy()
    assert got.shape == two.shape and np.array_equal(got, two)
    if x.size:
        red = int(np.prod([shape[a] for a in (axes or range(len(shape)))]))
        want = (x.astype(np.float64) ** 2).sum(axis=tuple(axes) if axes else None)
        assert_close(got, want, "sum of squares", scale=np.sqrt(red))
        # from a view one float off the 16-byte grid: the same bits (the order of the sums does not depend on alignment)
        whole = T(np.concatenate([[3.0], x.ravel()]).astype(np.float32))
        assert np.array_equal(ops.sum_of_squares(whole.view(1, shape), axes).numpy(), two)
        ax = sorted(axes or range(len(shape)))
        if ax == list(range(ax[0], ax[-1] + 1)):   # one run of adjacent axes: one pass (several runs have routes of their own)
            assert np.array_equal(ops.sum(whole.view(1, shape), axes).numpy(), ops.sum(T(x), axes).numpy())


def test_max_identity_is_minus_type_max():
    x = np.full((3, 5), -2**31, np.int32)
    assert np.array_equal(ops.max_element(T(x), (1,)).numpy(), O.max_element(x, (1,)))


@pytest.mark.parametrize("shape,axis", [((5,), 0), ((2, 3), 1), ((2, 3), 0), ((4, 5, 6), 1), ((3, 1000), 1),
                                        ((1000, 3), 0), ((37, 64), 1), ((300, 4097), 1), ((2, 3, 130), 2),
                                        ((64, 2048), 1), ((5, 256), 1), ((3, 1028), 1)])
def test_argmin(shape, axis):
    r = rng(12)
    x = r.integers(-5, 5, shape).astype(np.float32)   # many ties: first minimum must win
    got = ops.argmin(T(x), axis)
    assert got.dtype == np.int32
    assert np.array_equal(got.numpy(), O.argmin(x, axis))
    xi = r.integers(-5, 5, shape).astype(np.int32)
    assert np.array_equal(ops.argmin(T(xi), axis).numpy(), O.argmin(xi, axis))


def test_argmin_all_max_lane_gives_zero():
    x = np.full((2, 4), np.finfo(np.float32).max, np.float32)
    assert np.array_equal(ops.argmin(T(x), 1).numpy(), O.argmin(x, 1))
    # the wavefront-per-row kernel: rows that never fire, NaNs that never compare, a late first minimum
    x = np.full((4, 200), np.finfo(np.float32).max, np.float32)
    x[1, 150] = 1.0
    x[1, 199] = 1.0
    x[2, :] = np.nan
    x[3, :] = np.nan
    x[3, 70] = 5.0
    assert np.array_equal(ops.argmin(T(x), 1).numpy(), O.argmin(x, 1))


# ----------------------------------------------------------------------------- layout
@pytest.mark.parametrize("shape", [(7,), (4, 6), (3, 4, 5), (2, 3, 4, 5), (33, 65), (8388608 // 64 + 128,)])
def test_slice_pad_repeat(shape):
    r = rng(21)
    x = r.integers(-1000, 1000, shape).astype(np.int32)
    tx = T(x)
    for _ in range(3):
        start = [int(r.integers(0, s)) for s in shape]
        stop = [int(r.integers(a + 1, s + 1)) for a, s in zip(start, shape)]
        assert np.array_equal(ops.slice(tx, start, stop).numpy(), O.slice(x, start, stop))
        before = [int(r.integers(0, 3)) for _ in shape]
        after = [int(r.integers(0, 3)) for _ in shape]
        assert np.array_equal(ops.pad(tx, before, after).numpy(), O.pad(x, before, after))
    if x.size < 5000:
        reps = [int(r.integers(1, 4)) for _ in shape]
        assert np.array_equal(ops.repeat(tx, reps).numpy(), O.repeat(x, reps))
    # leading-axis slices are the batch-norm unpacking pattern (core/ops/nnet.d:484-488)
    cut = shape[0] // 2
    start, stop = [cut] + [0] * (len(shape) - 1), list(shape)
    assert np.array_equal(ops.slice(tx, start, stop).numpy(), x[cut:])


@pytest.mark.parametrize("shape,reps", [((4, 3, 8, 8), (1, 1, 2, 2)), ((6, 16), (3, 1)), ((5, 12), (1, 4)), ((2, 3, 4), (2, 1, 3)),
                                        ((128, 64), (1, 1)), ((7,), (5,))])
def test_repeat_quads_and_merged_axes(shape, reps):
    x = rng(23).integers(-1000, 1000, shape).astype(np.int32)
    assert np.array_equal(ops.repeat(T(x), list(reps)).numpy(), O.repeat(x, list(reps)))


def test_layout_maps_aligned_quads():
    """Extents, offsets and pointers that are all multiples of four take the 16-byte path."""
    x = rng(24).integers(-1000, 1000, (6, 5, 16)).astype(np.int32)
    tx = T(x)
    assert np.array_equal(ops.slice(tx, [1, 0, 4], [5, 5, 12]).numpy(), x[1:5, :, 4:12])
    assert np.array_equal(ops.pad(tx, [1, 0, 4], [0, 2, 8]).numpy(), O.pad(x, [1, 0, 4], [0, 2, 8]))
    assert np.array_equal(ops.pad(tx, [0, 0, 0], [0, 0, 128]).numpy(), O.pad(x, [0, 0, 0], [0, 0, 128]))


def test_slice_pad_large_index_range():
    """Above 2^27 elements the reciprocal-multiply quotient is off by one for many indices; the
    remainder correction has to catch every one of them."""
    shape = (5, 6151, 6143)
    x = np.arange(np.prod(shape), dtype=np.int64).astype(np.int32).reshape(shape)
    tx = T(x)
    got = ops.slice(tx, [1, 100, 141], [4, 6101, 6142]).numpy()
    assert np.array_equal(got, x[1:4, 100:6101, 141:6142])
    del got
    small = T(x[:3])
    got = ops.pad(small, [1, 0, 1], [0, 1, 0]).numpy()
    assert np.array_equal(got, np.pad(x[:3], ((1, 0), (0, 1), (1, 0))))


def test_slice_rejects_out_of_range():
    from dopt_amd import capi
    with pytest.raises(capi.HipError):
        ops.slice(T(np.zeros((3, 3), np.float32)), [1, 1], [4, 3])


@pytest.mark.parametrize("rows,cols", [(2, 2), (1, 9), (9, 1), (5, 9), (64, 64), (65, 130), (512, 512), (10, 784),
                                       (1000, 3),
                                       (68, 132), (4, 4), (4096, 2048), (100, 260), (8, 1028)])   # 128-bit tiles, ragged edges
def test_transpose(rows, cols):
    x = rng(22).standard_normal((rows, cols)).astype(np.float32)
    assert np.array_equal(ops.transpose(T(x)).numpy(), O.transpose(x))
    if rows % 4 == 0 and cols % 4 == 0 and rows * cols > 16:
        # an operand off the 16-byte grid takes the 32-bit tile kernel
        buf = T(np.concatenate([np.zeros(1, np.float32), x.ravel()]))
        assert np.array_equal(ops.transpose(buf.view(1, (rows, cols))).numpy(), O.transpose(x))


# ----------------------------------------------------------------------------- matmul
MM_SHAPES = [
    (2, 2, 1), (100, 10, 784), (784, 10, 100), (100, 10, 1), (1000, 1, 1), (100, 1, 10),      # config 1
    (256, 512, 784), (256, 512, 512), (256, 10, 512), (784, 512, 256), (256, 784, 512),        # config 2
    (128, 512, 512), (128, 10, 512), (128, 512, 1), (1, 512, 128), (512, 512, 128),            # VGG head
    (81920, 1, 64), (2359296, 1, 1),                                                           # WRN mean pool, scalar broadcast
    (7, 5, 3), (33, 65, 129), (130, 258, 70), (64, 256, 16), (65, 3, 200), (1, 17, 40), (19, 1, 23), (300, 300, 300),
]


@pytest.mark.parametrize("M,N,K", MM_SHAPES)
def test_matmul(M, N, K):
    r = rng(M * 31 + N * 7 + K)
    a = r.standard_normal((M, K)).astype(np.float32)
    b = r.standard_normal((K, N)).astype(np.float32)
    got = ops.matmul(T(a), T(b)).numpy()
    if K == 1:
        assert np.array_equal(got, a * b.reshape(1, N))      # a single rounding: exact
        return
    want = O.matmul(a, b, f64=True) if M * N * K < 5e8 else (a.astype(np.float64) @ b.astype(np.float64))
    assert_close(got, want, "matmul %dx%dx%d" % (M, N, K), scale=np.sqrt(K))
    # a dense layer's operands: He-scaled weights keep the products O(1); stated tolerance as it stands
    bw = (b * np.sqrt(2.0 / K)).astype(np.float32)
    want = O.matmul(a, bw, f64=True) if M * N * K < 5e8 else (a.astype(np.float64) @ bw.astype(np.float64))
    assert_close(ops.matmul(T(a), T(bw)).numpy(), want, "matmul, He-scaled %dx%dx%d" % (M, N, K))


def test_matmul_broadcast_by_ones_is_exact():
    # core/ops/basic.d:370-381: repeat(n) = ones[n,1] . x[1,vol]; scalars broadcast the same way
    x = rng(31).standard_normal((1, 513)).astype(np.float32)
    ones = np.ones((77, 1), np.float32)
    assert np.array_equal(ops.matmul(T(ones), T(x)).numpy(), np.repeat(x, 77, axis=0))
    s = np.array([[0.001]], np.float32)
    col = np.ones((100003, 1), np.float32)
    assert np.array_equal(ops.matmul(T(col), T(s)).numpy(), np.full((100003, 1), s[0, 0], np.float32))


def test_matmul_rejects_int():
    from dopt_amd import capi
    with pytest.raises(capi.HipError):
        ops.matmul(T(np.ones((2, 2), np.int32)), T(np.ones((2, 2), np.int32)))


# ----------------------------------------------------------------------------- convolution
CONV_CASES = [  # N, C, H, W, K, R, S, pad, stride
    (2, 3, 8, 8, 4, 3, 3, (1, 1), (1, 1)),
    (1, 2, 7, 9, 3, 3, 3, (0, 0), (1, 1)),
    (2, 2, 9, 8, 3, 3, 3, (1, 1), (2, 2)),
    (1, 3, 6, 6, 2, 1, 1, (0, 0), (2, 2)),
    (1, 1, 5, 7, 2, 2, 3, (1, 2), (1, 2)),
    (3, 16, 8, 8, 32, 3, 3, (1, 1), (1, 1)),
    (2, 20, 6, 6, 70, 3, 3, (1, 1), (1, 1)),      # channel counts that are not tile multiples
    (4, 3, 32, 32, 64, 3, 3, (1, 1), (1, 1)),     # VGG conv1 shape at batch 4
    (2, 64, 32, 32, 64, 3, 3, (1, 1), (1, 1)),    # VGG conv2
    (2, 64, 16, 16, 128, 3, 3, (1, 1), (1, 1)),   # VGG conv3
    (2, 128, 16, 16, 128, 3, 3, (1, 1), (1, 1)),  # VGG conv4
    (2, 128, 8, 8, 256, 3, 3, (1, 1), (1, 1)),    # VGG conv5
    (2, 256, 8, 8, 256, 3, 3, (1, 1), (1, 1)),    # VGG conv6-7
    (8, 256, 4, 4, 512, 3, 3, (1, 1), (1, 1)),    # VGG conv8: split reduction
    (8, 512, 4, 4, 512, 3, 3, (1, 1), (1, 1)),    # VGG conv9-10
    (16, 512, 2, 2, 512, 3, 3, (1, 1), (1, 1)),   # VGG conv11-13
    (2, 16, 32, 32, 160, 1, 1, (0, 0), (1, 1)),   # WRN 1x1 shortcut
    (2, 160, 32, 32, 320, 3, 3, (1, 1), (2, 2)),  # WRN stage entry, stride 2
    (2, 160, 32, 32, 320, 1, 1, (0, 0), (2, 2)),  # WRN strided shortcut
    # 3x3 unit-stride layers take the patch kernel: tiles of several whole images with a ragged
    # last tile, no padding / full padding (output smaller / larger than the input), channel counts
    # that are not multiples of 16, row counts that do not divide the tile (falls back to the gather)
    (5, 32, 4, 4, 130, 3, 3, (1, 1), (1, 1)),
    (3, 20, 8, 8, 70, 3, 3, (1, 1), (1, 1)),
    (2, 16, 10, 10, 40, 3, 3, (0, 0), (1, 1)),
    (2, 16, 6, 6, 24, 3, 3, (2, 2), (1, 1)),
    (2, 24, 16, 16, 64, 3, 3, (1, 0), (1, 1)),
    (1, 16, 12, 8, 32, 3, 3, (1, 1), (1, 1)),
    (3, 48, 2, 2, 200, 3, 3, (1, 1), (1, 1)),
    (130, 16, 2, 2, 16, 3, 3, (1, 1), (1, 1)),
    # filter-gradient patch kernel: rows of 8 / 16 / 32 / 64 pixels, both block shapes (K >= 128 or
    # not), channel counts off the 32-channel fragment, several bands per image, one-image batches
    (3, 40, 8, 8, 136, 3, 3, (1, 1), (1, 1)),
    (2, 70, 16, 16, 48, 3, 3, (1, 1), (1, 1)),
    (1, 33, 32, 32, 130, 3, 3, (1, 1), (1, 1)),
    (1, 16, 4, 64, 128, 3, 3, (1, 1), (1, 1)),
    (5, 96, 16, 8, 64, 3, 3, (1, 1), (1, 1)),
    (8, 40, 4, 4, 136, 3, 3, (1, 1), (1, 1)),     # 4x4 images, four per chunk
    (12, 64, 4, 4, 64, 3, 3, (1, 1), (1, 1)),
    (32, 48, 2, 2, 130, 3, 3, (1, 1), (1, 1)),    # 2x2 images, sixteen per chunk
    (16, 70, 2, 2, 32, 3, 3, (1, 1), (1, 1)),
    (6, 32, 4, 4, 128, 3, 3, (1, 1), (1, 1)),     # batch not a multiple of the chunk: generic kernel
    # 2x2 images at sizes whose filter gradient is one launch (dense product with the fold in its
    # epilogue): the VGG shape, and one with a shorter batch and ragged edge tiles
    (128, 512, 2, 2, 512, 3, 3, (1, 1), (1, 1)),
    # 2x2 images with channel counts in multiples of 64 read the filter itself (32 images x 8 channels per block, the
    # reduction split over its wavefronts): ragged tiles of images, one and three steps per wavefront
    (70, 64, 2, 2, 128, 3, 3, (1, 1), (1, 1)),
    (5, 192, 2, 2, 64, 3, 3, (1, 1), (1, 1)),
    (100, 500, 2, 2, 520, 3, 3, (1, 1), (1, 1)),
    # at most three input channels, pad 1: the first-layer kernels (rows of 8 .. 128 pixels, one to
    # sixteen rows per sub-tile, output channels off the 32-row fragment, a single-channel image)
    (3, 3, 32, 32, 40, 3, 3, (1, 1), (1, 1)),
    (2, 1, 16, 16, 8, 3, 3, (1, 1), (1, 1)),
    (5, 2, 16, 8, 33, 3, 3, (1, 1), (1, 1)),
    (2, 3, 4, 64, 64, 3, 3, (1, 1), (1, 1)),
    (1, 3, 3, 128, 20, 3, 3, (1, 1), (1, 1)),
    (7, 3, 24, 16, 64, 3, 3, (1, 1), (1, 1)),
    (2, 3, 28, 28, 16, 3, 3, (1, 1), (1, 1)),     # 28 is no power of two: general kernels
    (2, 3, 32, 32, 96, 3, 3, (1, 1), (1, 1)),     # more than 64 output channels: general kernels
    # strides: backward-data runs one residue class of pixels at a time (classes without a tap, uneven
    # class sizes, different strides per axis, a stride above the filter size, 5x5 filters)
    (2, 5, 9, 11, 7, 3, 3, (1, 1), (3, 3)),
    (3, 4, 10, 7, 6, 3, 3, (0, 1), (2, 1)),
    (2, 6, 8, 8, 5, 2, 2, (0, 0), (3, 3)),
    (1, 3, 13, 12, 4, 5, 5, (2, 2), (2, 2)),
    (2, 8, 7, 9, 3, 3, 2, (2, 0), (1, 2)),
    (4, 20, 16, 16, 36, 3, 3, (1, 1), (2, 2)),
    # the classes of a strided backward-data pass share one launch when there are two to four of them: 128-row tiles
    # with few tiles (eight wavefronts) and with many (four), odd extents (classes of different sizes)
    (2, 128, 8, 8, 64, 3, 3, (1, 1), (2, 2)),
    (16, 128, 64, 64, 16, 3, 3, (1, 1), (2, 2)),
    (3, 130, 9, 7, 24, 3, 3, (1, 1), (2, 2)),
    # Winograd F(2x2, 3x3): 128-row tiles of 32 2x2-pixel tiles - half an image, two images, eight images per tile;
    # a last tile with images missing; both directions (forward needs 128 k output channels, backward-data 128 k input
    # channels); a reduction split over workgroups
    (8, 128, 16, 16, 128, 3, 3, (1, 1), (1, 1)),
    (8, 128, 8, 8, 256, 3, 3, (1, 1), (1, 1)),
    (3, 64, 8, 8, 128, 3, 3, (1, 1), (1, 1)),
    (21, 256, 4, 4, 128, 3, 3, (1, 1), (1, 1)),
    (4, 128, 32, 32, 128, 3, 3, (1, 1), (1, 1)),
    # ... and 64-row tiles of 64 2x2-pixel tiles where the rows are whole 64s but not whole 128s: a quarter of an image,
    # one image, four images (the last tile with images missing), three row tiles
    (4, 64, 32, 32, 64, 3, 3, (1, 1), (1, 1)),
    (5, 128, 16, 16, 64, 3, 3, (1, 1), (1, 1)),
    (7, 64, 8, 8, 192, 3, 3, (1, 1), (1, 1)),
    (3, 192, 16, 16, 320, 3, 3, (1, 1), (1, 1)),
    (3, 160, 16, 16, 160, 3, 3, (1, 1), (1, 1)),   # 160 rows as three 64-row tiles, the last half empty
    (1, 80, 4, 4, 128, 3, 3, (1, 1), (1, 1)),      # one image in a tile of eight; five chunks (an odd count through two buffers)
    (5, 64, 8, 4, 128, 3, 3, (1, 1), (1, 1)),      # rows of four pixels, four images per tile
    (1, 64, 64, 64, 64, 3, 3, (1, 1), (1, 1)),     # 64-row tiles on rows of 64 pixels
    (2, 112, 16, 32, 128, 3, 3, (1, 1), (1, 1)),   # seven chunks, rows of 32 pixels
    (2, 80, 8, 12, 128, 3, 3, (1, 1), (1, 1)),     # 12 columns: no whole tile rows in 128 pixels, the direct kernels
    (2, 7, 11, 13, 9, 5, 5, (2, 2), (3, 3)),      # nine classes with work in one launch
    (1, 4, 9, 9, 5, 5, 5, (2, 2), (4, 4)),        # sixteen classes: one after the other
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_convolution_all_three(case):
    N, C, H, W, K, R, S, pad, st = case
    r = rng(hash(case) % 1000)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = (r.standard_normal((K, C, R, S)) * np.sqrt(2.0 / (C * R * S))).astype(np.float32)
    y_ref = O.convolution(x, w, pad, st)
    y = ops.convolution(T(x), T(w), pad, st)
    assert y.shape == y_ref.shape
    assert_close(y.numpy(), y_ref, "conv fwd", scale=1.0)
    dy = r.standard_normal(y_ref.shape).astype(np.float32)
    dx = ops.conv_bwd_data(T(dy), T(w), x.shape, pad, st).numpy()
    assert_close(dx, O.conv_bwd_data(dy, w, x.shape, pad, st), "conv bwd-data", scale=1.0)
    dw = ops.conv_bwd_filter(T(dy), T(x), w.shape, pad, st).numpy()
    npix = N * y_ref.shape[2] * y_ref.shape[3]
    assert_close(dw, O.conv_bwd_filter(dy, x, w.shape, pad, st), "conv bwd-filter", scale=np.sqrt(npix))
    # an upstream gradient with the 1/(pixels summed) scale of a mean loss: stated tolerance as it stands
    dys = (dy * np.float32(1.0 / npix)).astype(np.float32)
    dw = ops.conv_bwd_filter(T(dys), T(x), w.shape, pad, st).numpy()
    assert_close(dw, O.conv_bwd_filter(dys, x, w.shape, pad, st), "conv bwd-filter, mean-loss gradient")


@pytest.mark.parametrize("case", [(4, 3, 32, 32, 64), (4, 3, 16, 16, 16),      # first-layer kernels
                                  (4, 64, 16, 16, 128), (8, 128, 8, 8, 128),  # patch kernels
                                  (32, 128, 2, 2, 128), (3, 5, 7, 7, 6)])     # 2 x 2 images; the generic kernels
def test_convolution_operands_off_the_16_byte_grid(case):
    """Every operand and every result one float past a 16-byte boundary: kernels that load or store 128 bits at a
    time have to step aside (or handle it), and nothing may write outside its result."""
    N, C, H, W, K = case
    r = rng(N + C + H + K)
    x = r.standard_normal((N, C, H, W)).astype(np.float32)
    w = (r.standard_normal((K, C, 3, 3)) * np.sqrt(2.0 / (C * 9))).astype(np.float32)
    dy = r.standard_normal((N, K, H, W)).astype(np.float32)
    b = r.standard_normal(K).astype(np.float32)

    def off(a):   # the array one element into a buffer, with a guard element on either side
        t = T(np.concatenate([[7.0], a.ravel(), [7.0]]).astype(np.float32))
        return t, t.view(1, a.shape)

    def result(shape):
        t = T(np.full(int(np.prod(shape)) + 2, 7.0, np.float32))
        return t, t.view(1, shape)

    (_, xo), (_, wo), (_, dyo), (_, bo) = off(x), off(w), off(dy), off(b)
    pad, st = (1, 1), (1, 1)
    for name, want, run in (
            ("forward", O.convolution(x, w, pad, st), lambda o: ops.convolution(xo, wo, pad, st, out=o)),
            ("forward + bias", O.convolution(x, w, pad, st) + b[None, :, None, None],
             lambda o: ops.convolution_bias(xo, wo, bo, pad, st, out=o)),
            ("backward-data", O.conv_bwd_data(dy, w, x.shape, pad, st), lambda o: ops.conv_bwd_data(dyo, wo, x.shape, pad, st, out=o)),
            ("filter gradient", O.conv_bwd_filter(dy, x, w.shape, pad, st),
             lambda o: ops.conv_bwd_filter(dyo, xo, w.shape, pad, st, out=o))):
        whole, view = result(want.shape)
        run(view)
        got = whole.numpy()
        assert got[0] == 7.0 and got[-1] == 7.0, name
        assert_close(got[1:-1].reshape(want.shape), want, "%s %s" % (name, case), scale=np.sqrt(N * H * W) if "filter" in name else 1.0)


def test_convolution_matches_reference_cpu_kernel_on_same_shapes():
    # the reference CPU kernel (fp32, its own loop order) is a valid oracle when out dims == in dims
    r = rng(41)
    x = r.standard_normal((2, 8, 8, 8)).astype(np.float32)
    w = r.standard_normal((4, 8, 3, 3)).astype(np.float32)
    got = ops.convolution(T(x), T(w), (1, 1), (1, 1)).numpy()
    assert_close(got, O.convolution(x, w, (1, 1), (1, 1), f64=False), "conv vs cpu kernel", scale=np.sqrt(72))


# ----------------------------------------------------------------------------- pooling / softmax / relu / bias
@pytest.mark.parametrize("shape,dims", [((1, 1, 4, 4), (2, 2)), ((2, 3, 6, 9), (2, 3)), ((2, 3, 5, 5), (2, 2)),
                                        ((4, 64, 32, 32), (2, 2)), ((4, 512, 2, 2), (2, 2)), ((2, 3, 8, 6), (2, 2)),
                                        ((2, 2, 8, 8), (4, 2))])
def test_maxpool_and_grad(shape, dims):
    r = rng(51)
    x = r.integers(-3, 4, shape).astype(np.float32)    # ties everywhere: the tie rule is exercised
    y_ref = O.maxpool(x, dims)
    assert np.array_equal(ops.maxpool(T(x), dims).numpy(), y_ref)
    dy = r.standard_normal(y_ref.shape).astype(np.float32)
    assert np.array_equal(ops.maxpool_grad(T(dy), T(x), dims).numpy(), O.maxpool_grad(dy, x, dims))
    # NaNs: forward never selects one (acc < NaN is false), so backward must not route a gradient to one either
    xn = x.copy()
    xn.ravel()[::3] = np.nan
    yn = ops.maxpool(T(xn), dims).numpy()
    assert np.array_equal(yn, O.maxpool(xn, dims))
    gn = ops.maxpool_grad(T(dy), T(xn), dims).numpy()
    assert np.array_equal(gn, O.maxpool_grad(dy, xn, dims))
    ph, pw = dims
    P, Q = shape[2] // ph, shape[3] // pw
    win = xn[:, :, :P * ph, :Q * pw].reshape(shape[0], shape[1], P, ph, Q, pw)
    gw = gn[:, :, :P * ph, :Q * pw].reshape(shape[0], shape[1], P, ph, Q, pw)
    some_number = ~np.isnan(win).all(axis=(3, 5), keepdims=True)
    assert not (gw != 0)[np.isnan(win) & some_number].any()     # (an all-NaN window sends it to its first element)


@pytest.mark.parametrize("shape", [(1, 5), (128, 10), (256, 10), (4, 7, 3), (3, 5, 2, 2), (37, 64), (300, 1000),
                                   (5, 130), (70, 128), (9, 132), (33, 260), (17, 1024), (3, 1028), (1, 68), (6, 256), (6, 512), (6, 516)])
def test_softmax_and_grad(shape):
    r = rng(52)
    x = (r.standard_normal(shape) * 3).astype(np.float32)
    got = ops.softmax(T(x)).numpy()
    if len(shape) > 2 or shape[1] < 64:   # lane-per-row kernels: same loop order; expf differs by <= 2 ulp
        assert ulp_diff(got, O.softmax(x)).max() <= 4
    assert_close(got, O.softmax(x, f64=True), "softmax")
    y = O.softmax(x, f64=True)
    dy = r.standard_normal(shape).astype(np.float32)
    assert_close(ops.softmax_grad(T(dy), T(y)).numpy(), O.softmax_grad(dy, y), "softmax grad")


@pytest.mark.parametrize("n", [1, 5, 4096, 100003])
def test_relu(n):
    r = rng(53)
    x = r.standard_normal(n).astype(np.float32)
    x[::7] = 0.0
    if n > 2:
        x[2] = np.nan
    dy = r.standard_normal(n).astype(np.float32)
    got = ops.relu(T(x)).numpy()
    assert ulp_diff(got, O.relu(x)).max() == 0
    assert np.array_equal(ops.relu_grad(T(dy), T(x)).numpy(), O.relu_grad(dy, x))


@pytest.mark.parametrize("shape", [(4, 64, 32, 32), (3, 5, 4, 2), (6, 5), (128, 512, 2, 2), (2, 7, 3, 3),
                                   (64, 256, 8, 8)])
def test_bias(shape):
    r = rng(54)
    x = r.standard_normal(shape).astype(np.float32)
    b = r.standard_normal(shape[1]).astype(np.float32)
    assert np.array_equal(ops.add_bias(T(x), T(b)).numpy(), O.add_bias(x, b))
    red = x.size // shape[1]
    assert_close(ops.add_bias_grad(T(x)).numpy(), O.add_bias_grad(x), "bias grad", scale=np.sqrt(red))
    xs = (x * np.float32(1.0 / red)).astype(np.float32)
    assert_close(ops.add_bias_grad(T(xs)).numpy(), O.add_bias_grad(xs), "bias grad, mean-loss gradient")


# ----------------------------------------------------------------------------- batch norm
@pytest.mark.parametrize("shape", [(4, 3, 5, 5), (8, 6), (2, 4, 3, 1), (8, 64, 32, 32), (128, 512, 2, 2), (3, 2),
                                   (16, 16, 16, 16),
                                   (40, 4, 32, 32),     # channel too large for the register-resident path
                                   (128, 8, 16, 16),    # the largest channel that path takes (1024 threads)
                                   (5, 7, 4, 3),        # ragged tail in the resident path
                                   # two values per channel: xhat is +-1 up to eps, and dx is what is left of dy after
                                   # both projections cancel - O(eps / var) of dy, far below the absolute tolerance, so
                                   # a comparison relative to max|dx| reads large while the stated tolerance holds
                                   (2, 8, 1, 1), (2, 128, 1, 1), (2, 3, 1, 1), (2, 17, 1, 1)])
def test_batchnorm_train_grad_infer(shape):
    r = rng(61)
    C = shape[1]
    x = (r.standard_normal(shape) * 2 + 3).astype(np.float32)    # mean well away from 0
    gamma = r.standard_normal(C).astype(np.float32)
    beta = r.standard_normal(C).astype(np.float32)
    rm = r.standard_normal(C).astype(np.float32)
    rv = (r.random(C) + 0.5).astype(np.float32)
    dy = r.standard_normal(shape).astype(np.float32)
    mom = float(np.float32(0.9))
    vol = x.size
    m = vol // C
    got = ops.bn_train(T(x), T(gamma), T(beta), T(rm), T(rv), mom).numpy()
    want = O.bn_train(x, gamma, beta, rm, rv, mom)
    assert got.shape == (vol + 2 * C,)
    assert_close(got[:vol], want[:vol], "bn y")
    assert_close(got[vol:], want[vol:], "bn running stats")
    g = ops.bn_grad(T(dy), T(x), T(gamma)).numpy()
    gw = O.bn_grad(dy, x, gamma)
    assert_close(g[:vol], gw[:vol], "bn dx")
    assert_close(g[vol:], gw[vol:], "bn dscale/dbias", scale=np.sqrt(m))
    dys = (dy * np.float32(1.0 / m)).astype(np.float32)     # mean-loss scale: stated tolerance as it stands
    g = ops.bn_grad(T(dys), T(x), T(gamma)).numpy()
    gw = O.bn_grad(dys, x, gamma)
    assert_close(g[:vol], gw[:vol], "bn dx, mean-loss gradient")
    assert_close(g[vol:], gw[vol:], "bn dscale/dbias, mean-loss gradient")
    assert_close(ops.bn_infer(T(x), T(gamma), T(beta), T(rm), T(rv)).numpy(), O.bn_infer(x, gamma, beta, rm, rv),
                 "bn infer")


@pytest.mark.parametrize("shape", [(128, 64, 32, 32),    # the benchmark's largest channel: four blocks share one
                                   (130, 3, 32, 32),     # ragged pieces
                                   (33, 5, 16, 64),      # two pieces, the second much shorter than a full block
                                   (512, 2, 32, 32),     # the most blocks one channel may span
                                   (520, 1, 32, 32)])    # beyond that: the three-launch path
def test_batchnorm_channels_spanning_several_blocks(shape):
    """Channels of more than 32768 values: their statistics are combined across blocks.  Same checks as
    above plus the fused forms (ReLU on the way out, ReLU mask on the way in, per-channel sum of dx)."""
    import ctypes as C_
    from dopt_amd import capi
    lib = capi.load()
    r = rng(63)
    N, C = shape[:2]
    inner = shape[2] * shape[3]
    x = (r.standard_normal(shape) * 1.5 + 2).astype(np.float32)
    gamma, beta, rm = (r.standard_normal(C).astype(np.float32) for _ in range(3))
    rv = (r.random(C) + 0.5).astype(np.float32)
    vol, m = x.size, x.size // C
    dy = (r.standard_normal(shape) / m).astype(np.float32)
    mom = float(np.float32(0.9))
    tx, tg, tb, trm, trv, tdy = T(x), T(gamma), T(beta), T(rm), T(rv), T(dy)
    got = ops.bn_train(tx, tg, tb, trm, trv, mom).numpy()
    want = O.bn_train(x, gamma, beta, rm, rv, mom)
    assert_close(got[:vol], want[:vol], "bn y")
    assert_close(got[vol:], want[vol:], "bn running stats")
    fused = ops.bn_train_relu(tx, tg, tb, trm, trv, mom)
    assert np.array_equal(fused.numpy()[:vol], np.maximum(got[:vol], 0))
    assert np.array_equal(fused.numpy()[vol:], got[vol:])
    g = ops.bn_grad(tdy, tx, tg).numpy()
    gw = O.bn_grad(dy, x, gamma)
    assert_close(g[:vol], gw[:vol], "bn dx")
    assert_close(g[vol:], gw[vol:], "bn dscale/dbias")
    # relu mask on the way in, sum of dx on the way out
    y = fused.view(0, shape)
    packed, dxs = ops.Tensor((vol + 2 * C,)), ops.Tensor((C,))
    capi.check(lib.dopt_hip_bn_grad_fused(N, C, inner, tdy.ptr, y.ptr, tx.ptr, tg.ptr, packed.ptr, dxs.ptr))
    masked = O.relu_grad(dy, y.numpy())
    gw = O.bn_grad(masked, x, gamma)
    assert_close(packed.numpy()[:vol], gw[:vol], "bn dx behind a relu")
    assert_close(packed.numpy()[vol:], gw[vol:], "bn dscale/dbias behind a relu")
    assert_close(dxs.numpy(), O.add_bias_grad(packed.numpy()[:vol].reshape(shape)), "sum of dx")
    # twice the same call: the counters the blocks meet at are back at zero after every launch
    again = ops.bn_train(tx, tg, tb, trm, trv, mom).numpy()
    assert np.array_equal(again, got)
    ops.sync()


@pytest.mark.parametrize("shape", [(128, 8, 32, 32),    # four blocks per channel (the first pooled layer of the benchmark, fewer channels)
                                   (40, 4, 32, 32),     # two blocks per channel
                                   (35, 3, 30, 32),     # two blocks whose pieces split a pair of rows: pooled by a pass of its own
                                   (64, 6, 16, 16),     # one block, eight quads per lane
                                   (16, 5, 8, 8), (7, 3, 4, 4), (9, 4, 6, 4), (3, 2, 2, 128),   # one block, two quads per lane
                                   (16, 12, 2, 2),      # a quad is an image
                                   (5, 3, 4, 6), (4, 3, 4, 2), (6, 2, 6, 2), (2, 2, 2, 256)])   # shapes the resident kernels do not pool
def test_batchnorm_with_the_pool_behind_it(shape):
    """batchNormTrain + relu + maxpool [2,2] as one call and its gradient as one call: bit for bit the
    separate calls, which are the ones checked against the oracle; ties, zeros and NaNs in the windows."""
    r = rng(64)
    N, C, H, W = shape
    x = (r.standard_normal(shape) * 1.5 + 0.5).astype(np.float32)
    x[:, :, : H // 2 * 2 : 2, :] = np.round(x[:, :, : H // 2 * 2 : 2, :])     # plenty of equal values inside windows
    x[0, 0, 0, 0] = np.nan if N * H * W > 64 else x[0, 0, 0, 0]                # poisons channel 0 only
    gamma, beta, rm = (r.standard_normal(C).astype(np.float32) for _ in range(3))
    rv = (r.random(C) + 0.5).astype(np.float32)
    mom = float(np.float32(0.9))
    tx, tg, tb, trm, trv = T(x), T(gamma), T(beta), T(rm), T(rv)
    vol = x.size
    for relu in (True, False):
        sep = ops.bn_train_relu(tx, tg, tb, trm, trv, mom) if relu else ops.bn_train(tx, tg, tb, trm, trv, mom)
        sep_pool = ops.maxpool(sep.view(0, shape), (2, 2))
        packed, pooled = ops.bn_train_pool(tx, tg, tb, trm, trv, mom, relu=relu)
        assert np.array_equal(packed.numpy(), sep.numpy(), equal_nan=True), relu
        assert np.array_equal(pooled.numpy(), sep_pool.numpy(), equal_nan=True), relu
    # the oracle's view of the fused forward (channels without the NaN)
    want = O.bn_train(x[:, 1:], gamma[1:], beta[1:], rm[1:], rv[1:], mom)
    yo = O.relu(want[: x[:, 1:].size].reshape(x[:, 1:].shape))
    packed, pooled = ops.bn_train_pool(tx, tg, tb, trm, trv, mom)
    y = packed.view(0, shape)
    assert_close(y.numpy()[:, 1:], yo, "bn + relu y")
    assert np.array_equal(pooled.numpy()[:, 1:], O.maxpool(np.ascontiguousarray(y.numpy()[:, 1:]), (2, 2)))
    # gradient: dy of the pooled tensor at the scale a mean loss hands down
    dp = (r.standard_normal((N, C, H // 2, W // 2)) / (N * H * W)).astype(np.float32)
    tdp = T(dp)
    full = ops.maxpool_grad(tdp, y, (2, 2))
    sep, sep_sum = ops.Tensor((vol + 2 * C,)), ops.Tensor((C,))
    import ctypes as C_
    from dopt_amd import capi
    lib = capi.load()
    capi.check(lib.dopt_hip_bn_grad_fused(N, C, H * W, full.ptr, y.ptr, tx.ptr, tg.ptr, sep.ptr, sep_sum.ptr))
    dxs = ops.Tensor((C,))
    got = ops.bn_grad_pool(tdp, y, tx, tg, dx_sum=dxs)
    assert np.array_equal(got.numpy(), sep.numpy(), equal_nan=True)
    assert np.array_equal(dxs.numpy(), sep_sum.numpy(), equal_nan=True)
    got2 = ops.bn_grad_pool(tdp, y, tx, tg)      # without the sum of dx
    assert np.array_equal(got2.numpy(), sep.numpy(), equal_nan=True)
    # and against the oracle, composed operation by operation
    yh = np.ascontiguousarray(y.numpy()[:, 1:])
    gw = O.bn_grad(O.relu_grad(O.maxpool_grad(np.ascontiguousarray(dp[:, 1:]), yh, (2, 2)), yh),
                   np.ascontiguousarray(x[:, 1:]), gamma[1:])
    sub = x[:, 1:].size
    assert_close(got.numpy()[:vol].reshape(shape)[:, 1:].ravel(), gw[:sub], "bn dx behind relu and pool")
    assert_close(got.numpy()[vol + 1:vol + C], gw[sub:sub + C - 1], "bn dscale behind relu and pool")
    assert_close(got.numpy()[vol + C + 1:], gw[sub + C - 1:], "bn dbias behind relu and pool")
    ops.sync()


def test_batchnorm_blocks_that_do_not_meet_are_reported_and_recovered_from():
    """The blocks sharing a channel wait for each other a bounded number of polls.  With the bound at zero
    every block gives up at once (each still finishes and exits): the next synchronisation reports it, and
    with the bound restored the same call is correct again."""
    from dopt_amd import capi
    lib = capi.load()
    r = rng(64)
    shape = (128, 64, 32, 32)
    x = r.standard_normal(shape).astype(np.float32)
    ones, zeros = np.ones(64, np.float32), np.zeros(64, np.float32)
    tx, t1, t0 = T(x), T(ones), T(zeros)
    ops.sync()
    capi.check(lib.dopt_hip_bn_wait_limit(0))
    try:
        out = ops.bn_train(tx, t1, t0, t0, t1, 0.9)
        with pytest.raises(capi.HipError, match="did not meet"):
            ops.sync()
    finally:
        capi.check(lib.dopt_hip_bn_wait_limit(1 << 21))
    ops.sync()                                     # the error was reported once
    got = ops.bn_train(tx, t1, t0, t0, t1, 0.9, out=out).numpy()
    assert_close(got[:x.size], O.bn_train(x, ones, zeros, zeros, ones, 0.9)[:x.size], "bn y after recovery")


def test_batchnorm_large_mean_small_variance():
    # E[x^2] - E[x]^2 would lose everything here; the shifted moments must not
    r = rng(62)
    x = (1000.0 + r.standard_normal((64, 8, 16, 16)) * 0.01).astype(np.float32)
    ones, zeros = np.ones(8, np.float32), np.zeros(8, np.float32)
    got = ops.bn_train(T(x), T(ones), T(zeros), T(zeros), T(ones), 0.9).numpy()
    want = O.bn_train(x, ones, zeros, zeros, ones, 0.9)
    assert_close(got[:x.size], want[:x.size], "bn y, ill-conditioned", rtol=2e-3, atol=2e-3)
    assert_close(got[x.size + 8:], want[x.size + 8:], "running var", rtol=1e-3)


# ----------------------------------------------------------------------------- optimizers
def _opt_state(r, sizes):
    w = [r.standard_normal(n).astype(np.float32) for n in sizes]
    g = [(r.standard_normal(n) * 0.1).astype(np.float32) for n in sizes]
    m = [(r.standard_normal(n) * 0.1).astype(np.float32) for n in sizes]
    v = [np.abs(r.standard_normal(n) * 0.01).astype(np.float32) for n in sizes]
    vh = [np.abs(r.standard_normal(n) * 0.01).astype(np.float32) for n in sizes]
    return w, g, m, v, vh


OPT_SIZES = [1, 3, 4096, 4097, 10, 100003, 8192, 512]


@pytest.mark.parametrize("nesterov", [False, True])
def test_fused_sgd_is_bit_exact(nesterov):
    w, g, m, _, _ = _opt_state(rng(71), OPT_SIZES)
    tw, tg, tm = [T(a) for a in w], [T(a) for a in g], [T(a) for a in m]
    opt = ops.FusedOptimizer(tw, tg, tm)
    for step in range(2):
        opt.sgd(0.01, 0.9, nesterov)
        for i in range(len(w)):
            w[i], m[i] = O.sgd_step(w[i], g[i], m[i], 0.01, 0.9, nesterov)
    for i in range(len(w)):
        assert np.array_equal(tw[i].numpy(), w[i]) and np.array_equal(tm[i].numpy(), m[i]), i


@pytest.mark.parametrize("rule", ["adam", "amsgrad"])
def test_fused_adam_amsgrad_are_bit_exact(rule):
    w, g, m, v, vh = _opt_state(rng(72), OPT_SIZES)
    skip = [False] * len(w)
    skip[2] = True                                   # a projected parameter: w untouched, moments still updated
    w2_before = w[2].copy()
    tw, tg, tm, tv, tvh = ([T(a) for a in lst] for lst in (w, g, m, v, vh))
    opt = ops.FusedOptimizer(tw, tg, tm, tv, tvh if rule == "amsgrad" else None, skip)
    b1 = b2 = 1.0
    for step in range(3):
        getattr(opt, rule)(1e-3, 0.9, 0.999, 1e-8)
        b1, b2, eta = O.adam_scalars(1e-3, 0.9, 0.999, b1, b2)
        for i in range(len(w)):
            if rule == "adam":
                w[i], m[i], v[i] = O.adam_step(w[i], g[i], m[i], v[i], eta)
            else:
                w[i], m[i], v[i], vh[i] = O.amsgrad_step(w[i], g[i], m[i], v[i], vh[i], eta)
    assert opt.b1.value == np.float32(b1) and opt.b2.value == np.float32(b2)
    for i in range(len(w)):
        want_w = w2_before if skip[i] else w[i]
        assert np.array_equal(tw[i].numpy(), want_w), ("w", i)
        assert np.array_equal(tm[i].numpy(), m[i]), ("m", i)
        assert np.array_equal(tv[i].numpy(), v[i]), ("v", i)
        if rule == "amsgrad":
            assert np.array_equal(tvh[i].numpy(), vh[i]), ("vhat", i)


def test_batched_device_copies():
    import ctypes as C
    from dopt_amd import capi
    lib = capi.load()
    r = rng(90)
    sizes = [1, 3, 64, 512, 16384, 20000, 7, 100] * 8          # more than one launch's worth; one above 64 KiB
    src = [T(r.standard_normal(n).astype(np.float32)) for n in sizes]
    dst = [ops.Tensor((n,)) for n in sizes]
    n = len(sizes)
    d = (C.c_void_p * n)(*[t.ptr for t in dst])
    s = (C.c_void_p * n)(*[t.ptr for t in src])
    b = (C.c_size_t * n)(*[4 * k for k in sizes])
    capi.check(lib.dopt_hip_copy_d2d_batch(n, d, s, b))
    for a, c in zip(src, dst):
        assert np.array_equal(a.numpy(), c.numpy())
    # a chain a -> b -> c inside one call keeps its order
    a, bb, c = T(np.arange(8, dtype=np.float32)), ops.Tensor((8,)), ops.Tensor((8,))
    d = (C.c_void_p * 2)(bb.ptr, c.ptr)
    s = (C.c_void_p * 2)(a.ptr, bb.ptr)
    b = (C.c_size_t * 2)(32, 32)
    capi.check(lib.dopt_hip_copy_d2d_batch(2, d, s, b))
    assert np.array_equal(c.numpy(), np.arange(8, dtype=np.float32))
    # write-after-read inside one call: copy 1 reads `a`, copy 2 overwrites `a`; copy 1 must see the old `a`
    a, z, out = T(np.arange(8, dtype=np.float32)), T(np.full(8, 7, np.float32)), ops.Tensor((8,))
    d = (C.c_void_p * 2)(out.ptr, a.ptr)
    s = (C.c_void_p * 2)(a.ptr, z.ptr)
    capi.check(lib.dopt_hip_copy_d2d_batch(2, d, s, b))
    assert np.array_equal(out.numpy(), np.arange(8, dtype=np.float32))
    assert np.array_equal(a.numpy(), np.full(8, 7, np.float32))
    # a large copy (its own transfer) behind a small one whose destination it reads
    big = 20000
    a, m, out = T(np.arange(big, dtype=np.float32)), ops.Tensor((big,)), ops.Tensor((big,))
    head = T(np.full(8, -1, np.float32))
    capi.check(lib.dopt_hip_copy_d2d(m.ptr, a.ptr, 4 * big))
    d = (C.c_void_p * 2)(m.ptr, out.ptr)
    s = (C.c_void_p * 2)(head.ptr, m.ptr)
    b = (C.c_size_t * 2)(32, 4 * big)
    capi.check(lib.dopt_hip_copy_d2d_batch(2, d, s, b))
    want = np.arange(big, dtype=np.float32)
    want[:8] = -1
    assert np.array_equal(out.numpy(), want)


@pytest.mark.parametrize("shape", [(128, 512, 512), (70, 33, 129), (1024, 1024, 1024), (1, 300, 77), (200, 1, 64), (5, 7, 1)])
@pytest.mark.parametrize("tb", [False, True])
def test_sgemm_with_rank_one_term_and_relu(shape, tb):
    """dopt_hip_sgemm_rank1 (a dense layer in one kernel) against the four kernels it stands for, bit for
    bit: small-output kernel (epilogue in the kernel), tile engine and the matrix-vector / outer-product
    paths (epilogue as a pass of its own)."""
    M, N, K = shape
    r = rng(M + 5 * N + 11 * K + tb)
    a = T(r.standard_normal((M, K)).astype(np.float32))
    bh = r.standard_normal((K, N)).astype(np.float32)
    b = T(np.ascontiguousarray(bh.T) if tb else bh)
    u, v = T(r.standard_normal((M, 1)).astype(np.float32)), T(r.standard_normal((1, N)).astype(np.float32))
    prod = ops.matmul_t(a, b, False, tb)
    want = ops.pointwise("add", prod, ops.matmul(u, v))
    assert np.array_equal(ops.matmul_rank1(a, b, u, v, trans_b=tb).numpy(), want.numpy())
    assert np.array_equal(ops.matmul_rank1(a, b, u, v, relu=True, trans_b=tb).numpy(), ops.relu(want).numpy())
    assert np.array_equal(ops.matmul_rank1(a, b, None, None, relu=True, trans_b=tb).numpy(), ops.relu(prod).numpy())
    assert np.array_equal(ops.matmul_rank1(a, b, None, None, trans_b=tb).numpy(), prod.numpy())
    # and against the oracle
    ref = O.matmul(a.numpy(), bh, f64=True) + u.numpy().astype(np.float64) @ v.numpy().astype(np.float64)
    assert_close(ops.matmul_rank1(a, b, u, v, relu=True, trans_b=tb).numpy(), np.maximum(ref, 0), "sgemm_rank1", scale=np.sqrt(K))


@pytest.mark.parametrize("shape", [(2048, 2048, 128), (2048, 2048, 100), (2048, 2052, 17), (2044, 2080, 64)])
def test_sgemm_short_reduction_large_output(shape):
    # A stored [K][M], B stored [K][N], K <= 128 and about one 128 x 128 tile per CU: the kernel that
    # keeps both operand panels in LDS (full and ragged edge tiles, reductions that end inside a chunk)
    M, N, K = shape
    r = rng(M + 3 * N + 7 * K)
    a = r.standard_normal((M, K)).astype(np.float32)
    b = r.standard_normal((K, N)).astype(np.float32)
    got = ops.matmul_t(T(np.ascontiguousarray(a.T)), T(b), True, False)
    assert got.shape == (M, N)
    assert_close(got.numpy(), O.matmul(a, b, f64=True), "sgemm_t panel", scale=np.sqrt(K))


@pytest.mark.parametrize("shape", [(1024, 1024, 1024),   # 64 tiles, the reduction split over workgroups
                                   (2100, 2050, 36),     # more tiles than the small-output kernel takes, ragged edges
                                   (1100, 1030, 1026),   # a reduction that is no multiple of 4: element-wise loads
                                   (900, 1300, 515),     # ragged edges on both sides, odd reduction length
                                   (1600, 1500, 640),    # 128 x 128 tiles, the reduction split over workgroups
                                   (4096, 640, 70)])
def test_sgemm_large_products_all_operand_layouts(shape):
    """Products of more than 64 rows that the small-output kernel does not take (sgemm_rows_k): against float64, and
    every transposition - also with operands off the 16-byte grid - gives the product of the plain copies to the last
    bit (one order of summation per shape)."""
    M, N, K = shape
    r = rng(M + N + K)
    a = r.standard_normal((M, K)).astype(np.float32)
    b = (r.standard_normal((K, N)) * np.sqrt(2.0 / K)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    plain = ops.matmul(T(a), T(b)).numpy()
    assert_close(plain, want, "sgemm %dx%dx%d" % shape)
    for ta in (False, True):
        for tb in (False, True):
            sa, sb = (np.ascontiguousarray(a.T) if ta else a), (np.ascontiguousarray(b.T) if tb else b)
            assert np.array_equal(ops.matmul_t(T(sa), T(sb), ta, tb).numpy(), plain), (ta, tb)
            # the same operands one float off the 16-byte grid
            ba = T(np.concatenate([np.zeros(1, np.float32), sa.ravel()]))
            bb = T(np.concatenate([np.zeros(1, np.float32), sb.ravel()]))
            got = ops.matmul_t(ba.view(1, sa.shape), bb.view(1, sb.shape), ta, tb).numpy()
            assert np.array_equal(got, plain), (ta, tb, "unaligned")


@pytest.mark.parametrize("shape", [(12, 32768, 32), (32768, 12, 16), (12, 32768, 100), (64, 8192, 512), (8192, 64, 512),
                                   (33, 70000, 40), (70000, 33, 40), (128, 2048, 2048), (2048, 128, 2048),
                                   (256, 256, 8192), (1, 3000, 77), (3000, 1, 77), (1, 5000, 700), (5000, 1, 700),
                                   (40, 48, 300), (4096, 512, 128), (2100, 2050, 36), (100, 9, 1)])
def test_sgemm_order_names_what_gives_equal_bits(shape):
    """dopt_hip_sgemm_order's promise, which the plan's transpose folding rests on: whatever the flags, and whether a
    call computes the product or its transpose, calls with the same order value give the same bits.  At least the
    plain product and its transposed form with both flags set always exist; the count of differing values is
    printed by the assertion so that a shape whose every call stands alone is visible."""
    from dopt_amd import capi
    lib = capi.load()
    M, N, K = shape
    r = rng(M * 5 + N * 11 + K)
    a = r.standard_normal((M, K)).astype(np.float32)
    b = r.standard_normal((K, N)).astype(np.float32)
    seen = {}
    for out_t in (False, True):
        for ta in (False, True):
            for tb in (False, True):
                sa, sb = (np.ascontiguousarray(a.T) if ta else a), (np.ascontiguousarray(b.T) if tb else b)
                if out_t:   # (A B)^T = B^T A^T on the same memory: B as stored is B^T read transposed, and so on
                    order = lib.dopt_hip_sgemm_order(int(not tb), int(not ta), N, M, K)
                    got = ops.matmul_t(T(sb), T(sa), not tb, not ta).numpy().T
                else:
                    order = lib.dopt_hip_sgemm_order(int(ta), int(tb), M, N, K)
                    got = ops.matmul_t(T(sa), T(sb), ta, tb).numpy()
                assert order != 0
                if order in seen:
                    assert np.array_equal(got, seen[order][0]), (shape, (out_t, ta, tb), seen[order][1], hex(order))
                else:
                    seen[order] = (got, (out_t, ta, tb))
    assert len(seen) <= 4, sorted(hex(k) for k in seen)
    want = a.astype(np.float64) @ b.astype(np.float64)
    for got, which in seen.values():
        assert_close(got, want, "sgemm %s %s" % (shape, which), scale=np.sqrt(K))


@pytest.mark.parametrize("shape", [(128, 512, 512), (70, 33, 129), (130, 10, 512), (1, 300, 77), (200, 1, 64), (5, 7, 1),
                                   (256, 256, 40), (64, 260, 96)])
@pytest.mark.parametrize("ta,tb", [(False, True), (True, False), (True, True)])
def test_sgemm_transposed_operands(shape, ta, tb):
    M, N, K = shape
    r = rng(M * 7 + N * 3 + K)
    a = r.standard_normal((M, K)).astype(np.float32)
    b = r.standard_normal((K, N)).astype(np.float32)
    want = O.matmul(a, b, f64=True)
    got = ops.matmul_t(T(np.ascontiguousarray(a.T) if ta else a), T(np.ascontiguousarray(b.T) if tb else b), ta, tb)
    assert got.shape == (M, N)
    assert_close(got.numpy(), want, "sgemm_t", scale=np.sqrt(K))
    # on the matrix-core path it is the product of the transposed copies to the last bit (the
    # matrix-vector kernels sum in a different order when the matrix is read the other way)
    if min(M, N, K) > 1:
        assert np.array_equal(got.numpy(), ops.matmul(T(a), T(b)).numpy())


# ----------------------------------------------------------------------------- operands off the 16-byte grid
def _off(a):
    """(whole buffer, view one element in): the array with a guard element on either side."""
    t = T(np.concatenate([[7.0], np.asarray(a, np.float32).ravel(), [7.0]]).astype(np.float32))
    return t, t.view(1, np.shape(a))


@pytest.mark.parametrize("shape", [(8, 16, 8, 8), (16, 64, 32, 32), (4, 6, 6, 10), (64, 128, 2, 2)])
def test_entry_points_with_every_operand_off_the_16_byte_grid(shape):
    """Each tensor one float past a 16-byte boundary: the 128-bit kernels have to step aside, results equal those of
    the aligned call (to rounding where another kernel adds in another order), and nothing is written outside a result."""
    r = rng(sum(shape))
    N, Cc, H, W = shape
    x = r.standard_normal(shape).astype(np.float32)
    dy = r.standard_normal(shape).astype(np.float32)
    sc, bi = r.uniform(0.5, 1.5, Cc).astype(np.float32), r.standard_normal(Cc).astype(np.float32)
    rm, rv = r.standard_normal(Cc).astype(np.float32), r.uniform(0.5, 1.5, Cc).astype(np.float32)
    dp = r.standard_normal((N, Cc, H // 2, W // 2)).astype(np.float32)
    flat = x.reshape(N * Cc, H * W)
    n = x.size
    cases = [
        ("relu", (n,), lambda t, o: ops.relu(t(x), out=o)),
        ("reluGrad", (n,), lambda t, o: ops.relu_grad(t(dy), t(x), out=o)),
        ("addBias", shape, lambda t, o: ops.add_bias(t(x), t(bi), out=o)),
        ("addBiasGrad", (Cc,), lambda t, o: ops.add_bias_grad(t(dy), out=o)),
        ("maxpool", dp.shape, lambda t, o: ops.maxpool(t(x), (2, 2), out=o)),
        ("maxpoolGrad", shape, lambda t, o: ops.maxpool_grad(t(dp), t(x), (2, 2), out=o)),
        ("softmax", flat.shape, lambda t, o: ops.softmax(t(flat), out=o)),
        ("softmaxGrad", flat.shape, lambda t, o: ops.softmax_grad(t(dy.reshape(flat.shape)), t(np.abs(flat)), out=o)),
        ("batchNormTrain", (n + 2 * Cc,), lambda t, o: ops.bn_train(t(x), t(sc), t(bi), t(rm), t(rv), 0.9, out=o)),
        ("batchNormTrain+relu", (n + 2 * Cc,), lambda t, o: ops.bn_train_relu(t(x), t(sc), t(bi), t(rm), t(rv), 0.9, out=o)),
        ("batchNormGrad", (n + 2 * Cc,), lambda t, o: ops.bn_grad(t(dy), t(x), t(sc), out=o)),
        ("reluGrad+batchNormGrad", (n + 2 * Cc,), lambda t, o: ops.bn_grad_relu(t(dy), t(np.maximum(x, 0)), t(x), t(sc), out=o)),
        ("batchNormInference", shape, lambda t, o: ops.bn_infer(t(x), t(sc), t(bi), t(rm), t(rv), out=o)),
        ("sum over all", (), lambda t, o: ops.sum(t(x), None, out=o)),
        ("sum over [0,2,3]", (Cc,), lambda t, o: ops.sum(t(x), [0, 2, 3], out=o)),
        ("sum over [1]", (N, H, W), lambda t, o: ops.sum(t(x), [1], out=o)),
        ("maxElement over [2,3]", (N, Cc), lambda t, o: ops.max_element(t(x), [2, 3], out=o)),
        ("transpose", flat.shape[::-1], lambda t, o: ops.transpose(t(flat), out=o)),
        ("slice", (N, Cc, H - 1, W - 1), lambda t, o: ops.slice(t(x), [0, 0, 1, 0], [N, Cc, H, W - 1], out=o)),
        ("pad", (N, Cc, H + 1, W + 2), lambda t, o: ops.pad(t(x), [0, 0, 1, 1], [0, 0, 0, 1], out=o)),
        ("repeat", (N, Cc, 2 * H, W), lambda t, o: ops.repeat(t(x), [1, 1, 2, 1], out=o)),
        ("matmul", (N * Cc, N * Cc), lambda t, o: ops.matmul_t(t(flat), t(flat), False, True, out=o)),
    ]
    for name, oshape, run in cases:
        want = run(lambda a: T(np.asarray(a, np.float32)), None).numpy()
        size = int(np.prod(oshape)) if oshape != () else 1
        whole = T(np.full(size + 2, 7.0, np.float32))
        run(lambda a: _off(a)[1], whole.view(1, want.shape))
        got = whole.numpy()
        assert got[0] == 7.0 and got[-1] == 7.0, name
        assert_close(got[1:-1].reshape(want.shape), want, "%s %s" % (name, shape), scale=max(1.0, float(np.abs(want).max())))


def test_empty_tensors_are_no_ops_and_empty_folds_give_the_start_value():
    """Tensors without elements have no buffer (a 0-byte allocation is a null pointer): entry points take them as
    they are.  A reduction whose reduced axes are empty still fills its result, with the value the reference's fold
    starts from (cpu/math.d:183-187: 0 for sum, -T.max for maxElement)."""
    e = ops.Tensor((0, 4))
    assert ops.pointwise("add", e, ops.Tensor((0, 4))).shape == (0, 4)
    assert ops.relu(e).shape == (0, 4)
    assert np.array_equal(ops.sum(e, [0]).numpy(), np.zeros(4, np.float32))
    assert np.array_equal(ops.max_element(e, [0]).numpy(), np.full(4, -np.finfo(np.float32).max, np.float32))
    ei = ops.Tensor((3, 0), np.int32)
    assert np.array_equal(ops.sum(ei, [1]).numpy(), np.zeros(3, np.int32))
    assert np.array_equal(ops.max_element(ei, [1]).numpy(), np.full(3, -np.iinfo(np.int32).max, np.int32))
    assert ops.sum(e, [1]).shape == (0,)
    assert np.array_equal(ops.pad(e, [1, 0], [1, 0]).numpy(), np.zeros((2, 4), np.float32))
    assert ops.repeat(e, [2, 3]).shape == (0, 12)
    assert ops.matmul(ops.Tensor((3, 0)), ops.Tensor((0, 5))).numpy().tolist() == np.zeros((3, 5)).tolist()
    from dopt_amd import core
    a, b = core.float32([0, 4]), core.float32([0, 4])
    for flags in (0, core.PLAN_VIEWS | core.PLAN_FUSE):
        got = core.compile([a + b, core.sum(a * b), core.sum(a + b, [0])], flags).execute()
        assert got[0].shape == (0, 4) and got[1] == 0.0 and np.array_equal(got[2], np.zeros(4, np.float32))


@pytest.mark.parametrize("shape,axes", [((1000,), [0]), ((64, 300), [1]), ((64, 300), [0]), ((8, 16, 32), [0, 2]),
                                        ((5, 7), [0, 1]), ((100000,), [0]), ((33, 4096), [1])])
def test_max_element_passes_over_nans_like_the_reference_fold(shape, axes):
    """max(acc, x) = acc < x ? x : acc started at -T.max never takes a NaN (cpu/math.d:183-187): the result is the
    largest number, and -T.max where there is none.  In a tree of partial maxima a NaN must not hide the numbers
    it was paired with."""
    r = rng(len(shape) * 10 + axes[0])
    x = r.standard_normal(shape).astype(np.float32)
    x.ravel()[::7] = np.nan
    x.ravel()[:3] = np.nan
    want = O.max_element(x, axes)
    assert not np.isnan(want).any()
    assert np.array_equal(want, np.nanmax(x, axis=tuple(axes)))
    assert np.array_equal(ops.max_element(T(x), axes).numpy(), want)
    allnan = np.full(shape, np.nan, np.float32)
    got = ops.max_element(T(allnan), axes).numpy()
    assert np.array_equal(got, np.full(got.shape, -np.finfo(np.float32).max, np.float32))
    assert np.array_equal(got, O.max_element(allnan, axes))
