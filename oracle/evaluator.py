"""CPU evaluation of an operation graph with the oracle's kernels, in the order and with the kernels
of the reference's CPU evaluator (cpu/source/dopt/cpu/package.d:182-280: topological order, one
kernel per operation, variables read from `args` or from their own value).

TEST INFRASTRUCTURE ONLY, like the rest of this package: used by tests/ to check whole graphs that run
through HIPPlan against the CPU, and by the cpu_baseline leg of bench.py to time a configuration's
step on the host.  Operations the reference's CPU backend implements (cpu/math.d, cpu/basic.d,
cpu/nnet.d) use the fp32 restatements of those kernels (`ref_*`); the cuDNN-only operations, for which
the reference CPU evaluator throws (cpu/package.d:254-257), use the float64 direct loops (`f64_*`).

Graph nodes are duck-typed: anything with `opType`, `deps`, `attributes`, `shape`, `dtype` and, for
variables and constants, `value` (dopt_amd.core.Operation has them).
"""
import numpy as np

import oracle as O


def _topological(outputs):
    order, seen = [], set()
    for root in outputs:
        if id(root) in seen:
            continue
        seen.add(id(root))
        stack = [(root, 0)]
        while stack:
            op, i = stack[-1]
            if i < len(op.deps):
                stack[-1] = (op, i + 1)
                d = op.deps[i]
                if id(d) not in seen:
                    seen.add(id(d))
                    stack.append((d, 0))
            else:
                order.append(op)
                stack.pop()
    return order


def _transpose(x, order):
    if list(order) == list(range(x.ndim)):
        return x.copy()
    if x.ndim == 2:
        return O.transpose(x)                      # cpu/basic.d:117-153 handles rank 2 only, like the device backend
    raise NotImplementedError("transpose of rank %d" % x.ndim)


def _kernel(op, d, blas=False):
    t, a = op.opType, op.attributes
    if t in O.BINARY and len(d) == 2:
        return O.pointwise(t, d[0], d[1])
    if t in O.UNARY:
        return O.pointwise(t, d[0])
    if t == "matmul":
        # cpu/math.d:77-82 calls cblas gemm; `blas` times it that way (numpy's OpenBLAS at its default thread
        # count), the checker uses the plain loop whose order of summation is known
        return np.matmul(d[0], d[1]) if blas else O.matmul(d[0], d[1])
    if t == "sum":
        return O.sum(d[0], list(a["axes"]))
    if t == "maxElement":
        return O.max_element(d[0], list(a["axes"]))
    if t == "argmin":
        return O.argmin(d[0], int(a["axis"]))
    if t == "reshape":
        return d[0].reshape(op.shape)
    if t == "slice":
        return O.slice(d[0], list(a["start"]), list(a["stop"]))
    if t == "pad":
        return O.pad(d[0], list(a["before"]), list(a["after"]))
    if t == "repeat":
        return O.repeat(d[0], list(a["repetitions"]))
    if t == "transpose":
        return _transpose(d[0], a["order"])
    if t == "convolution":
        x, w = d
        same = all((x.shape[2 + i] + 2 * a["padding"][i] - w.shape[2 + i]) // a["stride"][i] + 1 == x.shape[2 + i]
                   for i in (0, 1))
        # the reference kernel (cpu/nnet.d:20-87) bounds its taps by the OUTPUT extents; where they differ
        # from the input's its result is not a convolution, and the float64 loops stand in
        return O.convolution(x, w, tuple(a["padding"]), tuple(a["stride"]), f64=not same)
    if t == "maxpool":
        return O.maxpool(d[0], tuple(a["dims"]))
    if t == "softmax":
        return O.softmax(d[0])
    # ---- no CPU kernel in the reference: float64 loops
    if t == "convolutionFeaturesGrad":
        return O.conv_bwd_data(d[0], d[1], tuple(a["featuresShape"]), tuple(a["padding"]), tuple(a["stride"]))
    if t == "convolutionFiltersGrad":
        return O.conv_bwd_filter(d[0], d[1], tuple(a["filtersShape"]), tuple(a["padding"]), tuple(a["stride"]))
    if t == "maxpoolGrad":
        return O.maxpool_grad(d[0], d[2], tuple(a["dims"]))
    if t == "softmaxGrad":
        return O.softmax_grad(d[0], d[1])
    if t == "relu":
        return O.relu(d[0])
    if t == "reluGrad":
        return O.relu_grad(d[0], d[2])
    if t == "addBias":
        return O.add_bias(d[0], d[1])
    if t == "addBiasGrad":
        return O.add_bias_grad(d[0])
    if t == "batchNormTrain":
        return O.bn_train(d[0], d[1].reshape(-1), d[2], d[3], d[4], float(a["momentum"]))
    if t == "batchNormGrad":
        # the reference judges this operation's type as volume(dy) + volume(x) + volume(scale) elements
        # (core/ops/nnet.d:232-235) although the kernel fills [dx | dscale | dbias]; the rest stays zero
        packed = O.bn_grad(d[0], d[1], d[2].reshape(-1))
        out = np.zeros(op.shape, np.float32)
        out.reshape(-1)[:packed.size] = packed
        return out
    if t == "batchNormInference":
        return O.bn_infer(d[0], d[1].reshape(-1), d[2], d[3], d[4])
    raise NotImplementedError("no CPU kernel for operation '%s'" % t)


def evaluate(outputs, args=None, blas=False):
    """Values of `outputs` (a list of graph nodes) as numpy arrays; args maps variables to arrays.  blas: matmul through
    the BLAS numpy links, as the reference's CPU backend calls cblas (for timing; not the checker's path)."""
    given = {id(k): np.ascontiguousarray(v, dtype=k.dtype).reshape(k.shape) for k, v in (args or {}).items()}
    vals = {}
    for op in _topological(list(outputs)):
        if op.opType in ("variable", "constant"):
            vals[id(op)] = given[id(op)] if id(op) in given else np.ascontiguousarray(op.value)
            continue
        out = _kernel(op, [vals[id(x)] for x in op.deps], blas)
        vals[id(op)] = np.ascontiguousarray(out).reshape(op.shape)
    return [vals[id(o)] for o in outputs]
