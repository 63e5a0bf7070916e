#!/usr/bin/env python3
"""Headline benchmark: one full training step (forward + backward + SGD update) of the VGG-16-style
CIFAR-shape network with batch norm at batch 128 in fp32, on one MI355X, through HIPPlan and the
kernel library.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config N] [--unfused] [--no-views] [--no-fuse]
                    [--graph] [--no-cpu] [--no-feed] [--no-kernel-timing]

A step is one execution of the update plan on device-resident synthetic inputs (inputs are in HBM
before the timed region starts).  W warm-up steps, then EXACTLY K timed steps between two device
synchronisations give `value`; four more windows of K steps give the median and the spread reported
beside it.  After the timed region the same step is run again with per-kernel HIP events (on the
library's stream, where the kernels are launched) to measure the dominant convolution kernel against
the fp32 MFMA roofline, and the reference's CPU path (this repository's C restatement of it) is timed
on the host cores as the reported CPU baseline.

--config 1|2|3|5 times one of the other configurations instead (a secondary line: they are parity
cases, not the headline); --config 4 is the default.
"""
import argparse
import json
import os
import statistics
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

BATCH = 128
MFMA_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0


def timed_windows(step, steps, warmup, windows=5):
    """W warm-up steps, then `windows` windows of exactly `steps` steps, each between two device
    synchronisations.  Returns seconds per window; the first is the official one."""
    from dopt_amd import ops
    step.run(warmup)
    ops.sync()
    out = []
    for _ in range(windows):
        t0 = time.perf_counter()
        step.run(steps)
        ops.sync()
        out.append(time.perf_counter() - t0)
    return out


def window_stats(win, steps):
    ms = [w / steps * 1e3 for w in win]
    return {"windows_ms_per_step": [round(m, 4) for m in ms], "median_ms_per_step": round(statistics.median(ms), 4),
            "spread_ms_per_step": round(max(ms) - min(ms), 4)}


def host_cores():
    try:
        return len(os.sched_getaffinity(0))
    except AttributeError:
        return os.cpu_count() or 1


def cpu_baseline(seconds_budget=20.0):
    """The reference's CPU path on the host cores (C restatement, `kind: port`):
      * the headline figure: its convolution kernel (cpu/source/dopt/cpu/nnet.d:20-87, single-threaded
        direct loops) over the 13 VGG layers at a small batch, as images/s of conv-forward alone -- the
        reference CPU backend has no backward, bias, ReLU or batch-norm kernels, so a CPU training step of
        the benchmark network does not exist;
      * configuration 1 (the one network the reference CPU backend can train end to end): whole training
        steps through the CPU evaluator, operation by operation in the reference's order."""
    import oracle as O
    from oracle import evaluator
    from dopt_amd import configs
    rng = np.random.default_rng(0)
    b = 1
    t_total = 0.0
    # calibrate on batch 1, then spend the remaining budget on one larger batch
    for attempt in range(2):
        t0 = time.perf_counter()
        for (c, k, h) in configs.VGG_CONVS:
            x = rng.standard_normal((b, c, h, h)).astype(np.float32)
            w = rng.standard_normal((k, c, 3, 3)).astype(np.float32)
            O.convolution(x, w, (1, 1), (1, 1), f64=False)
        t_total = time.perf_counter() - t0
        if attempt == 0:
            nb = int(max(1, min(32, (seconds_budget - t_total) / max(t_total, 1e-3))))
            if nb == b:
                break
            b = nb
    # configuration 1 on the CPU evaluator: graph outputs = loss, predictions, new W, new b, new momenta.  Timed twice:
    # every kernel on one thread, and threaded the way the reference's CPU backend is (matmul through BLAS at its
    # default thread count, cpu/math.d:77-82; sum / maxElement / repeat parallel over the outer index,
    # cpu/math.d:102,179, cpu/basic.d:166)
    s1 = configs.softmax_regression(flags=0, host_args=True)
    outs = s1.updater.plan.outputs

    def time_config1(blas):
        evaluator.evaluate(outs, s1.args, blas=blas)
        n, t0 = 0, time.perf_counter()
        while n < 3 or (time.perf_counter() - t0 < 2.0 and n < 200):
            evaluator.evaluate(outs, s1.args, blas=blas)
            n += 1
        return (time.perf_counter() - t0) / n * 1e3, n

    cfg1_ms, n1 = time_config1(False)
    cores = host_cores()
    O.set_threads(cores)
    try:
        cfg1_thr_ms, n1t = time_config1(True)
    finally:
        O.set_threads(1)
    try:
        from threadpoolctl import threadpool_info
        blas_threads = max([p.get("num_threads", 1) for p in threadpool_info() if p.get("user_api") == "blas"] or [1])
    except Exception:
        blas_threads = None
    return {"value": round(b / t_total, 3), "unit": "images/s", "cores": 1, "host_cores": cores, "kind": "port",
            "sample": "conv-forward only: the 13 VGG-16 3x3 convolutions at batch %d through the C restatement of "
                      "the reference's single-threaded CPU kernel (%.1f s; cpu/nnet.d:20-87 has no parallel loop); the "
                      "reference CPU backend implements no backward, bias, ReLU or batch-norm kernels, so a full CPU "
                      "training step does not exist" % (b, t_total),
            "config1_step_ms": round(cfg1_ms, 3),
            "config1_sample": "%d whole softmax-regression steps ([100,784] -> 10, forward + backward + SGD) through the "
                              "CPU evaluator, one restated reference kernel per operation, 1 thread" % n1,
            "config1_threaded_step_ms": round(cfg1_thr_ms, 3),
            "config1_threaded_cores": {"blas": blas_threads, "reductions_and_repeat": cores},
            "config1_threaded_sample": "%d of the same steps with the reference's own threading: matmul through OpenBLAS "
                                       "(numpy) at its default thread count, sum / maxElement / repeat parallel over "
                                       "the outer index on %d threads" % (n1t, cores)}


def host_feed_leg(step, steps, warmup):
    """The same step fed from host memory, as the reference's training loop runs it (examples/cifar10.d:118-140 fills
    float[] batches on the host; CUDAPlan.executeImpl uploads every host argument on each execution,
    cuda/package.d:367-401): a shuffled host dataset, mirrored-pad / random-crop / flip augmentation (ImageTransformer
    with 4, 4, true, false as in the example), page-locked staging and queued uploads through data.DeviceFeed, then the
    step.  Reported beside the headline figure, never as it."""
    from dopt_amd import data, ops, workloads
    rng = np.random.default_rng(3)
    n = 8 * BATCH
    X = rng.standard_normal((n, 3, 32, 32)).astype(np.float32)
    Y = workloads.one_hot(rng.integers(0, 10, n), 10)
    it = data.SupervisedBatchIterator(X, Y, [[3, 32, 32], [10]], shuffle=True, seed=4)
    feed = data.DeviceFeed(it, BATCH, 4, 4, True, False, seed=5)
    feats, labels = step.extra["feats"], step.extra["labels"]

    def run(k):
        for _ in range(k):
            if feed.finished():
                feed.restart()
            f, l = feed.next()
            step.updater.step_async({feats: f, labels: l})

    run(max(warmup, 2))
    ops.sync()
    t0 = time.perf_counter()
    run(steps)
    ops.sync()
    sec = (time.perf_counter() - t0) / steps
    # and the reference's own way: pageable host arrays handed to the plan, uploaded (blocking) inside every execution
    xs, ys = X[:BATCH].copy(), Y[:BATCH].copy()
    for _ in range(3):
        step.updater.step_async({feats: xs, labels: ys})
    ops.sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        step.updater.step_async({feats: xs, labels: ys})
    ops.sync()
    sec_plain = (time.perf_counter() - t0) / steps
    return {"ms_per_step": round(sec * 1e3, 4), "images_per_s": round(BATCH / sec, 1),
            "what": "the step with every batch coming from host memory: shuffled host dataset -> page-locked staging -> queued "
                    "upload on the second queue -> augmentation kernel (mirrored pad 4, random crop, horizontal flip) -> "
                    "training step; host fill and upload of batch k+1 overlap the device work of batch k",
            "pageable_args_ms_per_step": round(sec_plain * 1e3, 4),
            "pageable_args_what": "the same step with pageable numpy arrays as plan arguments, as examples/cifar10.d calls "
                                  "plan.execute: the plan stages them in page-locked memory of its own and uploads them on the "
                                  "second queue beside the previous execution (CUDAPlan.executeImpl uploads with a blocking copy)"}


def secondary(cfg, a):
    """One of the other configurations: a secondary JSON line."""
    from dopt_amd import configs, core
    flags = configs.REWRITES | (core.PLAN_GRAPH if a.graph else 0)
    if cfg == 1:
        step = configs.softmax_regression(flags=flags)
    elif cfg == 2:
        step = configs.mlp(fused=not a.unfused, flags=flags)
    elif cfg == 3:
        step = configs.fused_update("amsgrad" if a.unfused else "adam")
    else:
        step = configs.wide_resnet(BATCH, fused=not a.unfused, flags=flags)
    steps = a.steps if cfg != 5 else max(3, min(a.steps, 10))
    win = timed_windows(step, steps, a.warmup)
    sec = win[0] / steps
    res = {"metric": "secondary: training steps/sec of %s" % step.name, "value": round(1.0 / sec, 2), "unit": "steps/s",
           "n_gpus": 1, "steps": steps, "warmup": a.warmup, "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True,
           "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "config": {"workload": step.name, "plan_rewrites": "views+fuse" + ("+graph" if a.graph else "")}}
    res.update(window_stats(win, steps))
    if cfg == 3:
        res["roofline"] = {"kernel": "optim_k (fused multi-tensor update)", "bound": "hbm",
                           "achieved": round(step.extra["bytes_per_step"] / sec / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": round(step.extra["bytes_per_step"] / sec / 1e9 / HBM_PEAK_GBS, 4), "traffic": None}
    else:
        res["config"]["kernels_per_step"] = step.kernels()
        res["config"]["loss_after"] = round(step.loss_value(), 5)
    if cfg in (1, 2, 5):
        res["images_per_s"] = round(step.batch / sec, 1)
    if cfg == 5:
        fl = 3.0 * configs.wrn_conv_flops(BATCH)
        res["conv_TFLOPs"] = round(fl / sec / 1e12, 2)
        res["conv_flops_per_step"] = fl
    print(json.dumps(res))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=4, choices=[1, 2, 3, 4, 5])
    ap.add_argument("--unfused", action="store_true", help="run the reference's op-graph optimizer instead of the fused kernel")
    ap.add_argument("--no-views", action="store_true", help="disable the copy-eliding plan rewrites")
    ap.add_argument("--no-fuse", action="store_true", help="run every operation as its own kernel")
    ap.add_argument("--overlap", action="store_true", help="run the filter gradients on a second queue")
    ap.add_argument("--overlap-light", action="store_true",
                    help="run only the small steps off the main chain (dense-layer gradients) on a second queue")
    ap.add_argument("--graph", action="store_true", help="replay the step's kernels as a recorded HIP graph")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-feed", action="store_true", help="skip the host-fed variant of the step")
    ap.add_argument("--no-kernel-timing", action="store_true", help="skip the per-kernel event pass")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build drives one GPU per process and implements no collectives; run with --gpus 1")

    from dopt_amd import capi, configs, core, ops
    capi.check(capi.load().dopt_hip_init(0))
    if a.config != 4:
        return secondary(a.config, a)
    fused, views, fuse = not a.unfused, not a.no_views, not a.no_fuse

    def flags_for(timing):
        f = (core.PLAN_VIEWS if views else 0) | (core.PLAN_FUSE if (fuse and views) else 0)
        f |= (core.PLAN_TIMING | core.PLAN_TIMING_SHAPES) if timing else 0
        f |= core.PLAN_OVERLAP if a.overlap else 0
        f |= core.PLAN_OVERLAP_LIGHT if a.overlap_light else 0
        f |= core.PLAN_GRAPH if (a.graph and not timing) else 0
        return f

    step = configs.vgg16(BATCH, fused, flags_for(False))
    win = timed_windows(step, a.steps, a.warmup)
    elapsed = win[0]
    loss = step.loss_value()
    ms_per_step = elapsed / a.steps * 1e3
    stats = step.updater.plan.stats()

    result = {
        "metric": "train images/sec, VGG-16 CIFAR-shape fp32 b128",
        "value": round(BATCH / (elapsed / a.steps), 2),
        "unit": "images/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": step.name,
                   "global_batch": BATCH, "optimizer": "fused multi-tensor SGD" if fused else "op-graph SGD",
                   "plan_rewrites": ("views+fuse" if fuse else "views") if views else "none",
                   "kernels_per_step": stats["kernels"] + (1 if fused else 0),
                   "plan_buffer_MB": round(stats["buffer_bytes"] / 2**20, 1),
                   "parameters": int(sum(p.volume for p in step.params)), "loss_after": round(loss, 5)},
    }
    result.update(window_stats(win, a.steps))
    if not np.isfinite(loss):
        sys.exit("bench.py: the loss is not finite (%r)" % loss)
    if not a.no_feed:
        result["host_feed"] = host_feed_leg(step, a.steps, a.warmup)

    if not a.no_kernel_timing:
        # Same step, every kernel object bracketed by hipEvents on the library stream, keyed by operation
        # type and output shape.
        del step
        tstep = configs.vgg16(BATCH, fused, flags_for(True))
        tstep.run(2)
        ops.sync()
        before = tstep.updater.plan.profile()
        nsteps = max(3, min(a.steps, 10))
        lib = capi.load()
        capi.check(lib.dopt_hip_conv_pair_probe(2))      # events around every conv_wino_k launch, on its own stream
        tstep.run(nsteps)
        ops.sync()
        import ctypes as C
        pl, pus, pfl, pby = C.c_int(), C.c_double(), C.c_double(), C.c_double()
        capi.check(lib.dopt_hip_conv_pair_probe_read(C.byref(pl), C.byref(pus), C.byref(pfl), C.byref(pby)))
        capi.check(lib.dopt_hip_conv_pair_probe(0))
        after = tstep.updater.plan.profile()
        per_shape = {k: ((after[k][0] - before.get(k, (0, 0))[0]) / nsteps, (after[k][1] - before.get(k, (0, 0))[1]) // nsteps)
                     for k in after}
        per_op = {}
        for k, (us, n) in per_shape.items():
            name = k.split("@")[0]
            per_op[name] = (per_op.get(name, (0.0, 0))[0] + us, per_op.get(name, (0.0, 0))[1] + n)

        def profile_line(tag):
            """A figure of the committed rocprofv3 --pmc summary (FETCH_SIZE / WRITE_SIZE calibrated against a plain
            copy): NOT measured in this run."""
            tpath = os.path.join(ROOT, "profiles", "conv_kernels_vgg16_b128_hbm_traffic.txt")
            if os.path.exists(tpath):
                for line in open(tpath):
                    if line.startswith(tag + " "):
                        return int(line.split()[-1])
            return None

        def profile_kernel_avg(name):
            """Average duration (us) of a kernel in the committed rocprofv3 kernel-stats summary: NOT measured in this run."""
            spath = os.path.join(ROOT, "profiles", "vgg16_b128_train_step_kernel_stats.txt")
            if os.path.exists(spath):
                for line in open(spath):
                    if line.startswith(name + " "):
                        return float(line[len(name):].split()[2])
            return None

        # The dominant kernel, by its share of the step: conv_wino_k<16, 4, 1>, the Winograd F(2x2, 3x3) convolution on
        # 128-row tiles that runs the forward pass of layers 3-10 and the backward-data pass of layers 4-10 (15 launches
        # per step; the 64-row instantiation of layers 2-3 is not part of this figure).  Timed by events
        # recorded around each launch inside the library, on the stream the kernel runs on (its steps may also run a
        # split sum, which is not part of this figure).  `achieved` counts the layer's FLOPs by the direct algorithm,
        # 2*N*K*C*R*S*P*Q - the algorithmic work of the operation, as the other figures of this file do; the kernel
        # executes 16/36 of them on the matrix cores (`executed_*`), so `frac` above 1 is the algorithm's gain, not a
        # measurement error.
        launches = pl.value / nsteps if nsteps else 0
        tflops = pfl.value / (pus.value * 1e-6) / 1e12 if pus.value else 0.0
        result["roofline"] = {
            "kernel": "conv_wino_k<16, 4, 1>: Winograd F(2x2, 3x3) convolution on the transformed filter, 128 rows x 32 tiles of 2x2 "
                      "pixels per workgroup: forward of layers 3-10 and backward-data of layers 4-10 of the 13; the other "
                      "convolution kernels are listed under `kernels`",
            "bound": "mfma", "achieved": round(tflops, 2), "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(tflops / MFMA_FP32_PEAK_TFLOPS, 4),
            "executed_achieved": round(tflops * 16.0 / 36.0, 2), "executed_frac": round(tflops * 16.0 / 36.0 / MFMA_FP32_PEAK_TFLOPS, 4),
            "traffic": profile_line("traffic_bytes_per_launch conv_wino_k"),
            "traffic_source": "profiles/conv_kernels_vgg16_b128_hbm_traffic.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of "
                              "the same %d launches per step; taken from that file, not measured in this run)" % round(launches),
            "algorithmic_bytes_per_launch": int(pby.value / pl.value) if pl.value else None,
            "algorithmic_bytes_convention": "input, output and the filter once each",
            "launches_per_step": int(round(launches)),
            "flops_per_launch": round(pfl.value / pl.value, 1) if pl.value else None,
            "flops_convention": "2*N*K*C*R*S*P*Q per launch, the direct algorithm's count; the kernel's matrix instructions "
                                "execute 16/36 of it (sixteen products per 2x2 outputs instead of thirty-six)",
            "avg_launch_us": round(pus.value / pl.value, 2) if pl.value else None,
            "timing": "HIP events around each launch on the library's stream, %d steps; an event pair also sees the "
                      "boundary to the kernel in front (3-4 us), which the profiler's kernel durations do not" % nsteps,
            "profile_avg_launch_us": profile_kernel_avg("conv_wino_k<16, 4, 1>"),
            "profile_source": "profiles/vgg16_b128_train_step_kernel_stats.txt (rocprofv3 --kernel-trace --stats of this "
                              "command; taken from that file, not measured in this run)",
        }

        # The forward convolutions of layers 3-10 on their own (8 launches per step, the Winograd kernel): their steps
        # hold nothing else (filters are transformed by a step of their own; where a reduction is split the partial sums
        # are added by the batch norm behind it).
        flops = us = n128 = bytes_alg = 0
        for i, (c, k, h) in enumerate(configs.VGG_CONVS):
            fwd_keys = [n for n in ("convolution+addBias", "convolution") if "%s@%dx%dx%dx%d" % (n, BATCH, k, h, h) in per_shape]
            if h >= 4 and k >= 128 and fwd_keys:
                # forward layers sharing an output shape share a key: charge each layer its share
                same = sum(1 for (c2, k2, h2) in configs.VGG_CONVS if (k2, h2) == (k, h))
                t, n = per_shape["%s@%dx%dx%dx%d" % (fwd_keys[0], BATCH, k, h, h)]
                flops, us, n128 = flops + configs.conv_flops(BATCH, c, k, h), us + t / same, n128 + 1
                bytes_alg += 4 * (BATCH * c * h * h + BATCH * k * h * h + k * c * 9)     # input, output and filter once
        fwd = sum(configs.conv_flops(BATCH, c, k, h) for c, k, h in configs.VGG_CONVS)
        bwd_data = fwd - configs.conv_flops(BATCH, *configs.VGG_CONVS[0])
        conv_ops = ("convolution", "convolution+addBias", "convolutionFeaturesGrad", "convolutionFiltersGrad",
                    "convolutionFeaturesGrad+convolutionFiltersGrad", "filterPack")
        allconv_us = sum(per_op[k][0] for k in conv_ops if k in per_op)
        result["kernels"] = {
            "forward convolutions of layers 3-10 (conv_wino_k; FLOPs by the direct algorithm's count)": {
                "achieved_TFLOPs": round(flops / (us * 1e-6) / 1e12, 2) if us else None,
                "frac_of_mfma_peak": round(flops / (us * 1e-6) / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4) if us else None,
                "launches_per_step": n128, "avg_launch_us": round(us / n128, 2) if n128 else None,
                "algorithmic_bytes_per_launch": int(bytes_alg / n128) if n128 else None,
                "traffic": profile_line("traffic_bytes_per_launch conv_wino_k")},
            "all 38 convolution operations of the step incl. filter packing and split sums (2x2-image layers counted at the "
            "conventional 9-tap FLOPs although their dense route executes 4/9 of them)": {
                "achieved_TFLOPs": round((2 * fwd + bwd_data) / (allconv_us * 1e-6) / 1e12, 2),
                "frac_of_mfma_peak": round((2 * fwd + bwd_data) / (allconv_us * 1e-6) / 1e12 / MFMA_FP32_PEAK_TFLOPS, 4),
                "us_per_step": round(allconv_us, 1)},
            "device_us_per_step_by_op": {k: round(v[0], 1) for k, v in sorted(per_op.items(), key=lambda kv: -kv[1][0])},
            "device_us_per_step_total": round(sum(v[0] for v in per_op.values()), 1),
        }
        del tstep

    if not a.no_cpu:
        result["cpu_baseline"] = cpu_baseline()

    print(json.dumps(result))


if __name__ == "__main__":
    main()
