"""Host-side pieces of the feed path and the checkpoint format; no GPU.

ref_image_transform restates ImageTransformer.getBatch loop by loop; it is pinned here against
numpy's own symmetric padding, slicing and reversed views over every offset and flip of small images
(the reference holds no test for the class)."""
import numpy as np
import pytest

import oracle as O
from dopt_amd import core, data, nnet


@pytest.mark.parametrize("shape,jx,jy", [((2, 3, 5, 4), 2, 3), ((1, 1, 4, 4), 4, 4), ((2, 2, 6, 3), 0, 2), ((2, 2, 3, 6), 2, 0),
                                          ((3, 1, 2, 2), 0, 0)])
def test_oracle_image_transform_against_numpy_symmetric_pad(shape, jx, jy):
    x = np.random.default_rng(0).standard_normal(shape).astype(np.float32)
    n, _, h, w = shape
    p = np.pad(x, ((0, 0), (0, 0), (jy, jy), (jx, jx)), mode="symmetric")
    for xo in range(2 * jx + 1):
        for yo in range(2 * jy + 1):
            for flags in range(4):
                want = p[:, :, yo:yo + h, xo:xo + w]
                if flags & 1:
                    want = want[:, :, :, ::-1]
                if flags & 2:
                    want = want[:, :, ::-1, :]
                got = O.image_transform(x, jx, jy, [[xo, yo, flags]] * n)
                assert np.array_equal(got, want), (xo, yo, flags)


def test_oracle_image_transform_is_per_image():
    x = np.random.default_rng(1).standard_normal((4, 3, 8, 8)).astype(np.float32)
    geom = np.array([[0, 0, 0], [3, 1, 1], [2, 2, 2], [1, 3, 3]], np.int32)
    got = O.image_transform(x, 2, 2, geom)
    for i in range(4):
        assert np.array_equal(got[i:i + 1], O.image_transform(x[i:i + 1], 2, 2, geom[i:i + 1]))
    # offset (jitter, jitter) without flips is the identity
    assert np.array_equal(O.image_transform(x, 2, 2, [[2, 2, 0]] * 4), x)


def test_draw_geometry_ranges():
    g = data.draw_geometry(np.random.default_rng(0), 5000, 4, 2, True, False)
    assert g[:, 0].min() == 0 and g[:, 0].max() == 7      # uniform(0, 2 * jitter) excludes the upper end
    assert g[:, 1].min() == 0 and g[:, 1].max() == 3
    assert set(np.unique(g[:, 2])) == {0, 1}
    assert abs((g[:, 2] & 1).mean() - 0.5) < 0.05
    g = data.draw_geometry(np.random.default_rng(0), 100, 0, 0, False, True)
    assert not g[:, :2].any() and set(np.unique(g[:, 2])) == {0, 2}


def test_supervised_batch_iterator():
    feats = np.arange(10 * 6, dtype=np.float32).reshape(10, 6)
    labels = np.arange(10 * 2, dtype=np.float32).reshape(10, 2)
    it = data.SupervisedBatchIterator(feats, labels, [[1, 2, 3], [2]], shuffle=False)
    assert it.volume() == [6, 2] and it.length() == 10 and not it.finished()
    f, l = np.empty(4 * 6, np.float32), np.empty(4 * 2, np.float32)
    it.getBatch([f, l])
    assert np.array_equal(f, feats[:4].ravel()) and np.array_equal(l, labels[:4].ravel())
    it.getBatch([f, l])
    it.getBatch([f, l])                      # examples 8, 9 and zero fill
    assert np.array_equal(f[:12], feats[8:].ravel()) and not f[12:].any() and not l[4:].any()
    assert it.finished()
    it.restart()
    assert not it.finished()
    with pytest.raises(ValueError):
        it.getBatch([np.empty(7, np.float32), l])
    with pytest.raises(ValueError):
        data.SupervisedBatchIterator(feats, labels[:3], [[6], [2]], False)
    sh = data.SupervisedBatchIterator(feats, labels, [[6], [2]], shuffle=True, seed=3)
    sh.restart()
    f, l = np.empty(10 * 6, np.float32), np.empty(10 * 2, np.float32)
    sh.getBatch([f, l])
    order = (f.reshape(10, 6)[:, 0] / 6).astype(int)
    assert sorted(order) == list(range(10)) and list(order) != list(range(10))
    assert np.array_equal(l.reshape(10, 2), labels[order])     # features and labels stay paired


def test_checkpoint_format_is_raw_float32_in_parameter_order(tmp_path):
    init = nnet.Init(0)
    x = core.float32([2, 5])
    net = nnet.DAGNetwork([x], [nnet.dense(nnet.dense(nnet.dataSource(x), 4, init), 3, init)])
    path = tmp_path / "net.bin"
    net.save(path)
    raw = np.fromfile(path, "<f4")
    assert raw.size == 4 * 5 + 4 + 3 * 4 + 3
    want = np.concatenate([p.value.ravel() for p in net.params])
    assert np.array_equal(raw, want)
    for p in net.params:
        p.set_value(np.zeros(p.shape, np.float32))
    net.load(path)
    assert np.array_equal(np.concatenate([p.value.ravel() for p in net.params]), want)
    (tmp_path / "short.bin").write_bytes(raw[:10].tobytes())
    with pytest.raises(IOError):
        net.load(tmp_path / "short.bin")
