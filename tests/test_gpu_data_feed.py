"""The device side of the feed path: augmentation kernel against the oracle, page-locked staging,
and a checkpoint round trip through device-resident parameters."""
import numpy as np
import pytest

import oracle as O
from dopt_amd import capi, core, data, nnet, online, ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,jx,jy", [((128, 3, 32, 32), 4, 4), ((7, 1, 28, 28), 2, 0), ((5, 2, 9, 13), 0, 3), ((3, 3, 4, 4), 4, 4),
                                          ((2, 1, 1, 1), 0, 0), ((64, 3, 33, 31), 5, 7)])
def test_image_transform_matches_reference_loops(shape, jx, jy):
    r = np.random.default_rng(shape[0] * 7 + jx)
    x = r.standard_normal(shape).astype(np.float32)
    geom = np.stack([r.integers(0, 2 * jx + 1, shape[0]), r.integers(0, 2 * jy + 1, shape[0]), r.integers(0, 4, shape[0])],
                    1).astype(np.int32)
    got = data.image_transform(ops.tensor(x), jx, jy, ops.tensor(geom)).numpy()
    assert np.array_equal(got, O.image_transform(x, jx, jy, geom))


def test_image_transform_every_offset_and_flip():
    x = np.random.default_rng(2).standard_normal((1, 2, 5, 6)).astype(np.float32)
    cases = [(xo, yo, fl) for xo in range(5) for yo in range(7) for fl in range(4)]
    batch = np.repeat(x, len(cases), 0)
    geom = np.array(cases, np.int32)
    got = data.image_transform(ops.tensor(batch), 2, 3, ops.tensor(geom)).numpy()
    assert np.array_equal(got, O.image_transform(batch, 2, 3, geom))


def test_image_transform_argument_checks():
    t = ops.tensor(np.zeros((2, 1, 4, 4), np.float32))
    g = ops.tensor(np.zeros((2, 3), np.int32))
    with pytest.raises(capi.HipError):
        data.image_transform(t, 5, 0, g)          # a mirror wider than the image
    with pytest.raises(capi.HipError):
        data.image_transform(t, 1, 1, g, out=t)   # in place
    # offsets outside [0, 2 * jitter] are clamped to the image instead of read out of bounds
    wild = ops.tensor(np.array([[1000, -1000, 0], [-7, 9, 3]], np.int32))
    out = data.image_transform(t, 1, 1, wild).numpy()
    assert np.array_equal(out, np.zeros_like(out))


def test_pinned_staging_round_trip():
    a = data.PinnedArray([1000, 7])
    a.array[:] = np.arange(7000, dtype=np.float32).reshape(1000, 7)
    t = ops.Tensor([1000, 7])
    a.upload_async(t)
    assert np.array_equal(t.numpy(), a.array)      # numpy() waits for the queue
    with pytest.raises(capi.HipError):
        a.upload_async(ops.Tensor([3]))


def test_device_feed_produces_the_reference_batches():
    r = np.random.default_rng(0)
    feats = r.standard_normal((50, 3, 8, 8)).astype(np.float32)
    labels = np.eye(10, dtype=np.float32)[r.integers(0, 10, 50)]
    ds = data.SupervisedBatchIterator(feats, labels, [[3, 8, 8], [10]], shuffle=False)
    feed = data.DeviceFeed(ds, 16, jitter_x=2, jitter_y=2, flip_x=True, seed=11)
    twin = np.random.default_rng(11)                 # the same draws, replayed on the host
    seen = 0
    while not feed.finished():
        f, l = feed.next()
        geom = data.draw_geometry(twin, 16, 2, 2, True, False)
        raw = np.zeros((16, 3, 8, 8), np.float32)
        lab = np.zeros((16, 10), np.float32)
        k = min(16, 50 - seen)
        raw[:k], lab[:k] = feats[seen:seen + k], labels[seen:seen + k]
        assert np.array_equal(f.numpy(), O.image_transform(raw, 2, 2, geom))
        assert np.array_equal(l.numpy(), lab)
        seen += 16
    assert seen == 64


def test_checkpoint_round_trip_through_device_parameters(tmp_path):
    def make(seed):
        init = nnet.Init(seed)
        x, y = core.float32([8, 3, 8, 8]), core.float32([8, 4])
        top = nnet.dense(nnet.relu(nnet.batchNorm(nnet.conv2D(nnet.dataSource(x), 5, (3, 3), init, padding=(1, 1)))), 4, init)
        net = nnet.DAGNetwork([x], [top])
        return x, y, net, nnet.squaredError(top.trainOutput, y)

    r = np.random.default_rng(0)
    xs, ys = r.standard_normal((8, 3, 8, 8)).astype(np.float32), r.standard_normal((8, 4)).astype(np.float32)
    x, y, net, loss = make(1)
    up = online.fused_sgd([loss], net.params, net.paramProj, 0.05)
    for _ in range(3):
        up({x: xs, y: ys})
    trained = [p.value for p in net.params]            # read back from the device
    net.save(tmp_path / "ckpt.bin")

    x2, y2, net2, loss2 = make(2)                        # different initial values
    plan2 = core.compile([loss2])
    before, = plan2.execute({x2: xs, y2: ys})
    net2.load(tmp_path / "ckpt.bin")
    for a, p in zip(trained, net2.params):
        assert np.array_equal(a, p.value)
    after, = plan2.execute({x2: xs, y2: ys})             # the registered variables now hold the loaded values
    want, = core.compile([loss]).execute({x: xs, y: ys})
    assert after == want and after != before
