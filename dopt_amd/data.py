"""The feed path either side of the training step: batch iterators restating
nnet/source/dopt/nnet/data/package.d and imagetransformer.d, with the per-step work moved to the
device.

The reference fills pageable `float[]` batches on the host, augments them there one image at a
time, and uploads them with a blocking copy inside `plan.execute`.  Here a batch is written into
page-locked staging memory, queued to the device without waiting, augmented by one kernel, and
handed to the plan as device pointers; two staging/device buffer pairs alternate so that the host
fills batch k+1 while the device still trains on batch k.
"""
import ctypes as C

import numpy as np

from . import capi, ops


class BatchIterator:   # data/package.d:14-22
    def shape(self):
        raise NotImplementedError

    def volume(self):
        return [int(np.prod(s)) for s in self.shape()]

    def length(self):
        raise NotImplementedError

    def getBatch(self, batch_data):
        raise NotImplementedError

    def finished(self):
        raise NotImplementedError

    def restart(self):
        raise NotImplementedError


class SupervisedBatchIterator(BatchIterator):   # data/package.d:27-131
    def __init__(self, features, labels, shape, shuffle, seed=0):
        if len(features) != len(labels):
            raise ValueError("features.length != labels.length")
        if len(shape) == 0:
            raise ValueError("shape.length == 0")
        self._features = np.ascontiguousarray(features, np.float32).reshape(len(features), -1)
        self._labels = np.ascontiguousarray(labels, np.float32).reshape(len(labels), -1)
        self._shape = [list(s) for s in shape]
        self._shuffle = shuffle
        self._rng = np.random.default_rng(seed)
        self._indices = np.arange(len(features))
        self._front = 0

    def shape(self):
        return self._shape

    def length(self):
        return len(self._features)

    def finished(self):
        return self._front >= self.length()

    def restart(self):
        if self._shuffle:
            self._rng.shuffle(self._indices)
        self._front = 0

    def getBatch(self, batch_data):
        """Fills batch_data[0] (features) and batch_data[1] (labels), flat float32 arrays; a last
        batch that runs past the data is zero-filled, as in the reference."""
        vol = self.volume()
        if len(batch_data) != 2:
            raise ValueError("SupervisedBatchIterator.getBatch expects two arrays to fill.")
        f, l = (np.asarray(b).reshape(-1) for b in batch_data)
        if f.size % vol[0] != 0 or l.size % vol[1] != 0 or f.size // vol[0] != l.size // vol[1]:
            raise ValueError("batch arrays do not hold a whole number of examples")
        batch = f.size // vol[0]
        idx = self._indices[self._front:self._front + batch]
        f[:] = 0
        l[:] = 0
        f[:len(idx) * vol[0]] = self._features[idx].reshape(-1)
        l[:len(idx) * vol[1]] = self._labels[idx].reshape(-1)
        self._front += batch


class PinnedArray:
    """A float32 numpy view of page-locked host memory from the library."""

    def __init__(self, shape, dtype=np.float32):
        self.nbytes = int(np.prod(shape)) * np.dtype(dtype).itemsize
        p = C.c_void_p()
        capi.check(capi.load().dopt_hip_host_alloc(C.byref(p), self.nbytes))
        self.ptr = p.value
        buf = (C.c_char * self.nbytes).from_address(self.ptr)
        self.array = np.frombuffer(buf, dtype=dtype).reshape(shape)

    def upload_async(self, tensor, beside=False):
        """Queues the copy into `tensor`; the host must not refill this memory before the next sync.  `beside`: on the
        library's second queue, next to the work already queued instead of behind it (join with dopt_hip_upload_join)."""
        if tensor.nbytes != self.nbytes:
            raise capi.HipError(1, "Mismatch in buffer size")
        lib = capi.load()
        capi.check((lib.dopt_hip_copy_h2d_beside if beside else lib.dopt_hip_copy_h2d_async)(tensor.ptr, self.ptr, self.nbytes))

    def __del__(self):
        if getattr(self, "ptr", None):
            self.array = None
            try:
                capi.load().dopt_hip_host_free(self.ptr)
            except Exception:   # interpreter shutdown: the library may already be gone
                pass
            self.ptr = None


def draw_geometry(rng, n, jitter_x, jitter_y, flip_x, flip_y):
    """The per-image random draws of imagetransformer.d:96-97,112,120: crop offsets in
    [0, 2*jitter) (the reference's `uniform(0, 2 * jitter)` excludes the upper end) and two fair coins."""
    g = np.zeros((n, 3), np.int32)
    if jitter_x:
        g[:, 0] = rng.integers(0, 2 * jitter_x, n)
    if jitter_y:
        g[:, 1] = rng.integers(0, 2 * jitter_y, n)
    if flip_x:
        g[:, 2] |= (rng.random(n) < 0.5).astype(np.int32)
    if flip_y:
        g[:, 2] |= (rng.random(n) < 0.5).astype(np.int32) << 1
    return g


def image_transform(batch, jitter_x, jitter_y, geom, out=None):
    """Device tensors in, device tensor out: mirrored pad, crop and flips of a [N, C, H, W] batch;
    geom is an int32 [N, 3] device tensor of (xoff, yoff, flags)."""
    n, c, h, w = batch.shape
    out = out if out is not None else ops.Tensor(batch.shape)
    capi.check(capi.load().dopt_hip_image_transform(n, c, h, w, jitter_x, jitter_y, geom.ptr, batch.ptr, out.ptr))
    return out


class DeviceFeed:
    """ImageTransformer (imagetransformer.d:5-160) over a host iterator, producing device batches.

    next() returns (features, labels) device tensors for one batch.  The host side of batch k+1
    (iterator fill, random draws, staging) overlaps the device side of batch k: each of the two slots
    owns its staging memory and device buffers, and a slot is refilled only after the work the caller
    queued on it two calls ago has finished - found through an event recorded on entry to the call in
    between, so the host waits for that batch's step alone, not for the device to drain."""

    def __init__(self, dataset, batch_size, jitter_x=0, jitter_y=0, flip_x=False, flip_y=False, seed=0):
        self.dataset, self.batch = dataset, batch_size
        self.jx, self.jy, self.fx, self.fy = jitter_x, jitter_y, flip_x, flip_y
        self._rng = np.random.default_rng(seed)
        fshape, lshape = dataset.shape()
        if len(fshape) != 3:
            raise ValueError("image batches are [channels, height, width] per example")
        self._slots = []
        for _ in range(2):
            self._slots.append({
                "f_host": PinnedArray([batch_size] + list(fshape)), "l_host": PinnedArray([batch_size] + list(lshape)),
                "g_host": PinnedArray([batch_size, 3], np.int32),
                "raw": ops.Tensor([batch_size] + list(fshape)), "f": ops.Tensor([batch_size] + list(fshape)),
                "l": ops.Tensor([batch_size] + list(lshape)), "g": ops.Tensor([batch_size, 3], np.int32)})
        self._turn = 0
        self._marks = []
        for _ in range(2):
            ev = C.c_void_p()
            capi.check(capi.load().dopt_hip_event_create(C.byref(ev)))
            self._marks.append(ev)
        self._calls = 0

    def __del__(self):
        for ev in getattr(self, "_marks", []):
            try:
                capi.load().dopt_hip_event_destroy(ev)
            except Exception:   # interpreter shutdown
                pass
        self._marks = []

    def finished(self):
        return self.dataset.finished()

    def restart(self):
        self.dataset.restart()

    def next(self):
        s = self._slots[self._turn]
        self._turn ^= 1
        lib, j = capi.load(), self._calls
        self._calls += 1
        # the mark of the previous call lies behind everything queued before it, the step on this slot included
        if j >= 1:
            capi.check(lib.dopt_hip_event_sync(self._marks[(j - 1) & 1]))
        capi.check(lib.dopt_hip_event_record(self._marks[j & 1]))
        self.dataset.getBatch([s["f_host"].array, s["l_host"].array])
        s["g_host"].array[:] = draw_geometry(self._rng, self.batch, self.jx, self.jy, self.fx, self.fy)
        # The three uploads go to the second queue: the copy engine moves them while the first queue is still busy with
        # the step on the previous batch (nothing on the device reads this slot's buffers any more: the wait above).
        # The augmentation kernel, and whatever the caller queues next, waits for them.
        s["f_host"].upload_async(s["raw"], beside=True)
        s["l_host"].upload_async(s["l"], beside=True)
        s["g_host"].upload_async(s["g"], beside=True)
        capi.check(lib.dopt_hip_upload_join())
        image_transform(s["raw"], self.jx, self.jy, s["g"], out=s["f"])
        return s["f"], s["l"]
