"""Optimizers, in two forms.

`sgd`, `adam`, `amsgrad` restate online/source/dopt/online/{sgd,adam,amsgrad}.d: the update
rule is built as a graph of pointwise operations (scalars broadcast through products with ones
vectors) and compiled into one plan whose outputs are written back over the variables.  This is
the reference's own formulation; it runs on the HIP backend kernel by kernel and serves as the
un-fused ground truth.

`fused_sgd`, `fused_adam`, `fused_amsgrad` are what a `dopt.hip` build substitutes: the plan
computes only the outputs and the gradients (plus projections that do not depend on the updated
value, i.e. batch-norm's running statistics), and ONE multi-tensor kernel applies the rule in
place with the same per-node fp32 rounding, so parameters and optimizer state match the un-fused
form bit for bit.  Projections of the updated value itself (operator-norm constraints) run as a
second small plan after the kernel.
"""
import numpy as np

from . import capi, core, ops
from .core import float32, grad, sqrt


def _newbufs(variables):
    return [v.device_ptr()[0] for v in variables]


class _GraphUpdater:
    def __init__(self, outputs, plan_outputs, targets, flags):
        self.outputs = outputs
        self.plan = core.compile(plan_outputs, flags)
        self._targets = targets
        self._out_bufs = [ops.Tensor(o.shape, o.dtype) for o in outputs]
        self._rets = [t.ptr for t in self._out_bufs] + _newbufs(targets)

    def __call__(self, args=None):
        self.plan.execute(args, self._rets)
        return [t.numpy() for t in self._out_bufs]

    def step_async(self, args=None):
        """Enqueues one update without reading the outputs back."""
        self.plan.execute(args, self._rets)


def sgd(outputs, wrt, projs=None, learningRate=None, momentumRate=None, nesterov=False, flags=0):
    """online/sgd.d:28-94."""
    projs = projs or {}
    learningRate = learningRate if learningRate is not None else float32([], [0.01])
    momentumRate = momentumRate if momentumRate is not None else float32([], [0.0])
    grads = grad(outputs[0], wrt)
    momentum = [float32(g.shape) for g in grads]
    if nesterov:
        new_momentum = [m * momentumRate - learningRate * g for g, m in zip(grads, momentum)]
        newvals = [w + momentumRate * nm - learningRate * g for w, nm, g in zip(wrt, new_momentum, grads)]
    else:
        new_momentum = [m * momentumRate + learningRate * g for g, m in zip(grads, momentum)]
        newvals = [w - nm for w, nm in zip(wrt, new_momentum)]
    for i, w in enumerate(wrt):
        if w in projs:
            newvals[i] = projs[w](newvals[i])
    up = _GraphUpdater(outputs, list(outputs) + newvals + new_momentum, list(wrt) + momentum, flags)
    up.momentum = momentum
    return up


def _adam_graph(outputs, wrt, projs, alpha, beta1, beta2, eps, with_varhat, flags):
    projs = projs or {}
    alpha = alpha if alpha is not None else float32([], [0.001])
    beta1 = beta1 if beta1 is not None else float32([], [0.9])
    beta2 = beta2 if beta2 is not None else float32([], [0.999])
    eps = eps if eps is not None else float32([], [1e-8])
    grads = grad(outputs[0], wrt)
    means = [float32(w.shape) for w in wrt]
    vars_ = [float32(w.shape) for w in wrt]
    varhats = [float32(w.shape) for w in wrt] if with_varhat else []
    b1, b2 = float32([], [1.0]), float32([], [1.0])
    nb1, nb2 = b1 * beta1, b2 * beta2
    eta = alpha * sqrt(1.0 - nb2) / (1.0 - nb1)
    new_means = [beta1 * m + (1.0 - beta1) * g for g, m in zip(grads, means)]
    new_vars = [beta2 * v + (1.0 - beta2) * g * g for g, v in zip(grads, vars_)]
    new_varhats = [core.max(vh, v) for vh, v in zip(varhats, vars_)]
    newvals = [w - eta * (m / (sqrt(v) + eps)) for w, m, v in zip(wrt, new_means, new_vars)]
    for i, w in enumerate(wrt):
        if w in projs:
            newvals[i] = projs[w](newvals[i])
    up = _GraphUpdater(outputs, list(outputs) + newvals + new_means + new_vars + new_varhats + [nb1, nb2],
                       list(wrt) + means + vars_ + varhats + [b1, b2], flags)
    up.means, up.vars, up.varhats, up.b1, up.b2 = means, vars_, varhats, b1, b2
    return up


def adam(outputs, wrt, projs=None, alpha=None, beta1=None, beta2=None, eps=None, flags=0):
    """online/adam.d:32-93."""
    return _adam_graph(outputs, wrt, projs, alpha, beta1, beta2, eps, False, flags)


def amsgrad(outputs, wrt, projs=None, alpha=None, beta1=None, beta2=None, eps=None, flags=0):
    """online/amsgrad.d:32-99."""
    return _adam_graph(outputs, wrt, projs, alpha, beta1, beta2, eps, True, flags)


# ------------------------------------------------------------------------------- fused

class _Placeholder:
    pass


class _FusedUpdater:
    def __init__(self, rule, outputs, wrt, projs, hyper, flags):
        projs = projs or {}
        self.rule, self.hyper, self.outputs, self.wrt = rule, hyper, list(outputs), list(wrt)
        grads = grad(outputs[0], wrt)
        # Three kinds of projection (online/sgd.d:75-85 applies them to the updated value inside
        # the one plan):
        #  - it ignores the updated value (batch-norm replaces its running statistics by graph
        #    outputs, nnet/layers/batchnorm.d:140-154): computed by the step's plan, the kernel skips
        #    the parameter;
        #  - it depends on the updated value and otherwise on nothing the step reads (the
        #    operator-norm projections of nnet/lipschitz.d: constants, their own scalar variables,
        #    fresh random draws): a second plan, run after the fused kernel, reads the updated
        #    parameter and writes the projected one over it;
        #  - it also reads other variables (the max-gain projections read this batch's
        #    activations, computed from the OLD parameters): only the op-graph optimizers can
        #    reproduce that ordering.
        proj_ops, skip, post = [], [], []
        step_nodes = {id(o) for o in core.topological_sort(list(outputs))}   # what the step itself reads
        for w in wrt:
            skip.append(False)
            if w not in projs:
                continue
            probe = float32(w.shape)
            p = projs[w](probe)
            nodes = core.topological_sort([p])
            if not any(o is probe for o in nodes):
                proj_ops.append((w, p))
                skip[-1] = True
            elif all(o is probe or o.opType != "variable" or id(o) not in step_nodes for o in nodes):
                post.append((w, projs[w](w)))
            else:
                raise NotImplementedError("fused updaters cannot order a projection that reads both the updated "
                                          "value and other variables; use dopt_amd.online.%s for this model" % rule)
        self._post_plan = core.compile([p for _, p in post], flags) if post else None
        self._post_rets = [w.device_ptr()[0] for w, _ in post]
        self._proj = proj_ops
        self.plan = core.compile(list(outputs) + grads + [p for _, p in proj_ops], flags)
        self._out_bufs = [ops.Tensor(o.shape, o.dtype) for o in outputs]
        self._rets = [t.ptr for t in self._out_bufs] + [None] * len(grads) + [w.device_ptr()[0] for w, _ in proj_ops]

        def view(op_or_var, ptr):
            return ops.Tensor(op_or_var.shape, np.float32, _ptr=ptr, _owner=self)

        params = [view(w, w.device_ptr()[0]) for w in wrt]
        gviews = [view(g, self.plan.result_ptr(g)[0]) for g in grads]
        self.state = {"m": [ops.Tensor(w.shape) for w in wrt]}
        if rule in ("adam", "amsgrad"):
            self.state["v"] = [ops.Tensor(w.shape) for w in wrt]
        if rule == "amsgrad":
            self.state["vhat"] = [ops.Tensor(w.shape) for w in wrt]
        self.opt = ops.FusedOptimizer(params, gviews, self.state["m"], self.state.get("v"), self.state.get("vhat"),
                                      skip)

    def step_async(self, args=None):
        # The plan reads the OLD parameters; the fused kernel then updates them in place; projected
        # parameters were written by the plan's return copies (they are skipped by the kernel).
        self.plan.execute(args, self._rets)
        h = self.hyper
        if self.rule == "sgd":
            self.opt.sgd(h["lr"], h["mu"], h["nesterov"])
        elif self.rule == "adam":
            self.opt.adam(h["alpha"], h["beta1"], h["beta2"], h["eps"])
        else:
            self.opt.amsgrad(h["alpha"], h["beta1"], h["beta2"], h["eps"])
        if self._post_plan is not None:
            self._post_plan.execute(None, self._post_rets)

    def __call__(self, args=None):
        self.step_async(args)
        return [t.numpy() for t in self._out_bufs]


def fused_sgd(outputs, wrt, projs=None, learningRate=0.01, momentumRate=0.0, nesterov=False, flags=0):
    return _FusedUpdater("sgd", outputs, wrt, projs,
                         {"lr": float(learningRate), "mu": float(momentumRate), "nesterov": bool(nesterov)}, flags)


def fused_adam(outputs, wrt, projs=None, alpha=0.001, beta1=0.9, beta2=0.999, eps=1e-8, flags=0):
    return _FusedUpdater("adam", outputs, wrt, projs,
                         {"alpha": float(alpha), "beta1": float(beta1), "beta2": float(beta2), "eps": float(eps)},
                         flags)


def fused_amsgrad(outputs, wrt, projs=None, alpha=0.001, beta1=0.9, beta2=0.999, eps=1e-8, flags=0):
    return _FusedUpdater("amsgrad", outputs, wrt, projs,
                         {"alpha": float(alpha), "beta1": float(beta1), "beta2": float(beta2), "eps": float(eps)},
                         flags)
