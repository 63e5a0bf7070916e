"""Per-kernel throughput of the bandwidth-bound entry points against the HBM roofline.

    python -m dopt_amd.kernel_bench [--iters 50] [--scale S] [--json]

Each row times one C-ABI entry point at a shape taken from the benchmark configurations (the
VGG-16 b128 activations, the 16M-parameter fused update) with HIP events on the library's stream
and reports ALGORITHMIC bytes / time: every tensor counted once per kernel, whatever the kernel
really moves (a two-pass batch norm reads its input twice but is charged 8 B/element).  At the
configuration shapes (33.5 MB per tensor) a kernel lasts 5-15 us, of which 2-3 us are launch ramp
and tail; --scale S multiplies the leading dimension of every shape by S to show the rate the same
kernels reach on tensors that take longer to stream.
"""
import argparse
import ctypes as C
import json

import numpy as np

from . import capi, ops, workloads

HBM_PEAK = 8.0e12
MFMA_FP32_PEAK = 157.3e12

# [M, K] x [K, N] products: cubes, the dense layers of the MLP configuration (forward and the two gradient
# products of the widest layer), and the dense form of a 3x3 convolution over 2x2 images at batch 128
GEMM_SHAPES = [(1024, 1024, 1024), (2048, 2048, 2048), (4096, 4096, 4096), (8192, 8192, 8192),
               (256, 512, 784), (256, 512, 512), (256, 10, 512), (784, 512, 256), (256, 784, 512),
               (128, 2048, 2048), (2048, 2048, 128)]


def gemm_rows():
    """(M, N, K, seconds-callable) per product, C = A . B through dopt_hip_sgemm."""
    rows, keep = [], []
    for (M, N, K) in GEMM_SHAPES:
        a, b = _rand((M, K), 11), _rand((K, N), 12)
        o = ops.matmul(a, b)
        keep += [a, b, o]
        rows.append((M, N, K, (lambda a=a, b=b, o=o: ops.matmul(a, b, out=o))))
    return rows, keep


_blocker = []


def _hold_the_queue():
    """Enqueues a product that lasts several milliseconds.  The calls timed behind it are enqueued while it runs, so
    the device executes them back to back and the events measure kernels, not the host's call overhead (a Python call
    into the library costs as much as a short kernel lasts)."""
    if not _blocker:
        a, b = _rand((8192, 8192), 21), _rand((8192, 8192), 22)
        _blocker.extend([a, b, ops.matmul(a, b)])
    ops.matmul(_blocker[0], _blocker[1], out=_blocker[2])


def _time(fn, iters, warm=5):
    lib = capi.load()
    ev = [C.c_void_p(), C.c_void_p()]
    for e in ev:
        capi.check(lib.dopt_hip_event_create(C.byref(e)))
    for _ in range(warm):
        fn()
    _hold_the_queue()
    capi.check(lib.dopt_hip_event_record(ev[0]))
    for _ in range(iters):
        fn()
    capi.check(lib.dopt_hip_event_record(ev[1]))
    ms = C.c_float()
    capi.check(lib.dopt_hip_event_elapsed_ms(ev[0], ev[1], C.byref(ms)))
    for e in ev:
        lib.dopt_hip_event_destroy(e)
    return ms.value * 1e-3 / iters


def _rand(shape, seed=0):
    return ops.tensor(np.random.default_rng(seed).standard_normal(shape, dtype=np.float32))


def cases(scale=1):
    """(name, shape text, algorithmic bytes, callable) per row.  Every callable writes into an output
    tensor allocated once, before the timed loop, so a row times the kernels of one entry point only."""
    rows, keep = [], []

    def add(name, shape, nbytes, fn):
        o = fn(None)                                         # the first call allocates the output ...
        keep.append(o)
        rows.append((name, shape, nbytes, lambda: fn(o)))   # ... every later call reuses it

    act = (128 * scale, 64, 32, 32)              # the largest VGG activation: 8.39 M elements, 33.5 MB
    n = int(np.prod(act))
    x, dy = _rand(act, 1), _rand(act, 2)
    fa, fb = x.reshape((n,)), dy.reshape((n,))
    add("pointwise add", "%d" % n, 12 * n, lambda o: ops.pointwise("add", fa, fb, out=o))
    add("pointwise mul", "%d" % n, 12 * n, lambda o: ops.pointwise("mul", fa, fb, out=o))
    add("pointwise abs", "%d" % n, 8 * n, lambda o: ops.pointwise("abs", fa, out=o))
    add("pointwise exp", "%d" % n, 8 * n, lambda o: ops.pointwise("exp", fa, out=o))
    add("relu", str(act), 8 * n, lambda o: ops.relu(x, out=o))
    add("reluGrad", str(act), 12 * n, lambda o: ops.relu_grad(dy, x, out=o))
    bias = _rand((64,), 3)
    add("addBias", str(act), 8 * n, lambda o: ops.add_bias(x, bias, out=o))
    add("addBiasGrad", str(act), 4 * n, lambda o: ops.add_bias_grad(dy, out=o))
    add("maxpool 2x2", str(act), 5 * n, lambda o: ops.maxpool(x, (2, 2), out=o))
    pdy = _rand((128 * scale, 64, 16, 16), 4)
    add("maxpoolGrad 2x2", str(act), 9 * n, lambda o: ops.maxpool_grad(pdy, x, (2, 2), out=o))
    g, b, rm, rv = (_rand((64,), 5 + i) for i in range(4))
    rv.set(np.abs(rv.numpy()) + 0.5)
    add("batchNormTrain", str(act), 8 * n, lambda o: ops.bn_train(x, g, b, rm, rv, 0.9, out=o))
    add("batchNormGrad", str(act), 12 * n, lambda o: ops.bn_grad(dy, x, g, out=o))
    add("batchNormInference", str(act), 8 * n, lambda o: ops.bn_infer(x, g, b, rm, rv, out=o))
    # the same pair with the 2x2 max-pool of a VGG block riding along: y and its pooled quarter written by one
    # launch; backward, dy made from the pooled tensor's gradient on the way in (dp, y, x read; dx written)
    ybuf = ops.bn_train_relu(x, g, b, rm, rv, 0.9)
    yv = ybuf.view(0, act)
    pooled = ops.Tensor((act[0], 64, 16, 16))
    add("batchNormTrain+relu+maxpool", str(act), 9 * n, lambda o: ops.bn_train_pool(x, g, b, rm, rv, 0.9, out=o, pooled=pooled)[0])
    add("maxpoolGrad+reluGrad+batchNormGrad", str(act), 13 * n, lambda o: ops.bn_grad_pool(pdy, yv, x, g, out=o))
    add("sum (all axes)", str(act), 4 * n, lambda o: ops.sum(x, out=o))
    add("sum axes [0,2,3]", str(act), 4 * n, lambda o: ops.sum(x, [0, 2, 3], out=o))
    add("maxElement (all axes)", str(act), 4 * n, lambda o: ops.max_element(x, out=o))
    m2 = x.reshape((4096 * scale, 2048))
    add("transpose", str(tuple(m2.shape)), 8 * n, lambda o: ops.transpose(m2, out=o))
    add("argmin axis 1", str(tuple(m2.shape)), 4 * n, lambda o: ops.argmin(m2, 1, out=o))
    sm = _rand((65536 * scale, 128), 9)
    add("softmax", str(tuple(sm.shape)), 8 * sm.size, lambda o: ops.softmax(sm, out=o))
    add("slice (contiguous)", "%d -> %d" % (n, n - 128), 8 * (n - 128), lambda o: ops.slice(fa, [0], [n - 128], out=o))
    add("slice (4-d interior)", "%s -> (.., 30, 30)" % (act,), 8 * act[0] * 64 * 900,
        lambda o: ops.slice(x, [0, 0, 1, 1], [act[0], 64, 31, 31], out=o))
    add("pad (1-d tail)", "%d + 128" % n, 8 * n, lambda o: ops.pad(fa, [0], [128], out=o))
    add("repeat", "%s x [1,1,2,2]" % (act,), 20 * n, lambda o: ops.repeat(x, [1, 1, 2, 2], out=o))

    # the fused multi-tensor updates over the 16 777 216-parameter, 40-tensor workload
    st = workloads.adam16m_state(0)
    tw, tg, tm, tv, tvh = ([ops.tensor(s[k]) for s in st] for k in ("w", "g", "m", "v", "vhat"))
    total = workloads.ADAM16M_TOTAL
    sgd = ops.FusedOptimizer(tw, tg, tm)
    adam = ops.FusedOptimizer(tw, tg, tm, tv)
    ams = ops.FusedOptimizer(tw, tg, tm, tv, tvh)
    rows.append(("fused SGD (40 tensors)", "%d" % total, 20 * total, lambda: sgd.sgd(0.01, 0.9, False)))
    rows.append(("fused ADAM (40 tensors)", "%d" % total, 28 * total, lambda: adam.adam(1e-3, 0.9, 0.999, 1e-8)))
    rows.append(("fused AMSGrad (40 tensors)", "%d" % total, 36 * total, lambda: ams.amsgrad(1e-3, 0.9, 0.999, 1e-8)))
    keep.extend([x, dy, bias, pdy, g, b, rm, rv, sm, tw, tg, tm, tv, tvh, sgd, adam, ams, ybuf, yv, pooled])
    return rows, keep


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--iters", type=int, default=50)
    ap.add_argument("--scale", type=int, default=1, help="multiply the leading dimension of the activation shapes")
    ap.add_argument("--json", action="store_true")
    ap.add_argument("--gemm", action="store_true", help="the fp32 matrix products against the MFMA roofline instead")
    args = ap.parse_args()
    if args.gemm:
        rows, keep = gemm_rows()
        res = []
        for M, N, K, fn in rows:
            sec = _time(fn, args.iters)
            res.append({"M": M, "N": N, "K": K, "us": sec * 1e6, "TFLOP/s": 2.0 * M * N * K / sec / 1e12,
                        "frac_of_157.3": 2.0 * M * N * K / sec / MFMA_FP32_PEAK})
        ops.sync()
        if args.json:
            print(json.dumps(res))
            return
        print("%-28s %10s %10s %8s" % ("matmul [M,K] x [K,N]", "us", "TFLOP/s", "of peak"))
        for r in res:
            print("%-28s %10.1f %10.1f %7.1f%%" % ("[%d,%d] x [%d,%d]" % (r["M"], r["K"], r["K"], r["N"]), r["us"], r["TFLOP/s"],
                                                    100 * r["frac_of_157.3"]))
        return
    out = []
    rows, keep = cases(args.scale)
    for name, shape, nbytes, fn in rows:
        sec = _time(fn, args.iters)
        out.append({"kernel": name, "shape": shape, "us": sec * 1e6, "GB/s": nbytes / sec / 1e9,
                    "frac_of_8TB/s": nbytes / sec / HBM_PEAK})
    ops.sync()
    if args.json:
        print(json.dumps(out))
        return
    print("%-28s %-40s %10s %10s %8s" % ("kernel", "shape", "us", "GB/s", "of peak"))
    for r in out:
        print("%-28s %-40s %10.1f %10.0f %7.1f%%" % (r["kernel"], r["shape"], r["us"], r["GB/s"], 100 * r["frac_of_8TB/s"]))


if __name__ == "__main__":
    main()
