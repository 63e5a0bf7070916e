"""Host-side mirror of the part of dopt.core a backend is driven by: Operation graphs, the op
constructors with their verifiers and shape judges, reverse-mode `grad`, and `evaluate` /
`compile` dispatching to the HIP backend's plan.

In a deployment this layer is the reference's own D code (core/source/dopt/core), used
unchanged; it is restated here only so that tests and the benchmark can build exactly the graphs
the reference builds (same op names, dependency order, attribute keys and shapes) and hand them
to HIPPlan through the C ABI.  No arithmetic on tensor data happens in this file.

Citations are to core/source/dopt/core/ of the reference.
"""
import builtins
import ctypes as C

import numpy as np

from . import capi

_bmax = builtins.max   # several reference op names (max, min, sum, abs, pow, slice) shadow builtins below
float32_t = np.dtype(np.float32)
int32_t = np.dtype(np.int32)
_CODE = {float32_t: capi.F32, int32_t: capi.I32}


def _vol(shape):
    v = 1
    for s in shape:
        v *= int(s)
    return v


class VerificationError(Exception):
    """ops/package.d:240-242: 'Operation of type "..." failed verification.'"""


# ------------------------------------------------------------------------------- graph container

class _DeviceGraph:
    """The one process-wide dopt_hip graph that Operations are registered into on first use."""

    def __init__(self):
        self.handle = None
        self.generation = 0

    def get(self):
        if self.handle is None:
            h = C.c_void_p()
            capi.check(_lib().dopt_hip_graph_create(C.byref(h)))
            self.handle = h
        return self.handle


_graph = _DeviceGraph()
_plan_api_ready = False


def _lib():
    global _plan_api_ready
    lib = capi.load()
    if not _plan_api_ready:
        sz, vp, i = C.c_size_t, C.c_void_p, C.c_int
        protos = {
            "dopt_hip_graph_create": [C.POINTER(vp)],
            "dopt_hip_graph_destroy": [vp],
            "dopt_hip_graph_add_op": [vp, C.c_char_p, i, i, C.POINTER(sz), i, C.POINTER(i), C.POINTER(i)],
            "dopt_hip_graph_set_attr_sizes": [vp, i, C.c_char_p, C.POINTER(sz), i],
            "dopt_hip_graph_set_attr_double": [vp, i, C.c_char_p, C.c_double],
            "dopt_hip_graph_value": [vp, i, C.POINTER(vp), C.POINTER(sz)],
            "dopt_hip_graph_op_type": [vp, i, C.POINTER(C.c_char_p), C.POINTER(i), C.POINTER(i), C.POINTER(sz),
                                       C.POINTER(i)],
            "dopt_hip_graph_op_dep": [vp, i, i, C.POINTER(i)],
            "dopt_hip_register_kernel": [C.c_char_p, vp, vp],
            "dopt_hip_deregister_kernel": [C.c_char_p],
            "dopt_hip_list_operations": [C.c_char_p, sz, C.POINTER(sz)],
            "dopt_hip_plan_create": [vp, i, C.POINTER(i), C.c_uint, C.POINTER(vp)],
            "dopt_hip_plan_execute": [vp, i, C.POINTER(i), C.POINTER(vp), C.POINTER(i), i, C.POINTER(vp)],
            "dopt_hip_plan_result": [vp, i, C.POINTER(vp), C.POINTER(sz)],
            "dopt_hip_plan_stats": [vp, C.POINTER(sz), C.POINTER(sz)],
            "dopt_hip_plan_recordings": [vp, C.POINTER(sz), C.POINTER(sz)],
            "dopt_hip_plan_profile": [vp, C.c_char_p, sz, C.POINTER(sz)],
            "dopt_hip_plan_destroy": [vp],
        }
        for name, argtypes in protos.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = C.c_int
        _plan_api_ready = True
    return lib


PLAN_SYMBOLS = ["dopt_hip_graph_create", "dopt_hip_graph_destroy", "dopt_hip_graph_add_op",
                "dopt_hip_graph_set_attr_sizes", "dopt_hip_graph_set_attr_double", "dopt_hip_graph_value",
                "dopt_hip_graph_op_type", "dopt_hip_graph_op_dep", "dopt_hip_register_kernel",
                "dopt_hip_deregister_kernel", "dopt_hip_list_operations", "dopt_hip_plan_create",
                "dopt_hip_plan_execute", "dopt_hip_plan_result", "dopt_hip_plan_stats", "dopt_hip_plan_recordings", "dopt_hip_plan_profile",
                "dopt_hip_plan_destroy"]


# ------------------------------------------------------------------------------- Operation

_OPDEFS = {}   # name -> (verifier, judge)   ops/package.d:253-258
_GRADS = {}    # name -> gradient function   grads/package.d:131-141


def register_operation(name, verifier, judge):
    if name in _OPDEFS:
        raise ValueError("There is already an operation registered with the name '%s'" % name)
    _OPDEFS[name] = (verifier, judge)


def register_gradient(name, fn):
    if name in _GRADS:
        raise ValueError("A gradient is already registered for operation '%s'" % name)
    _GRADS[name] = fn


class Operation:
    """A node in the expression graph (ops/package.d:52-251)."""

    def __init__(self, op_type, deps=(), attributes=None):
        if op_type not in _OPDEFS:
            raise KeyError("Cannot create operation because there is no operation definition registered with the "
                           "name '%s'" % op_type)
        self.opType = op_type
        self.deps = list(deps)
        self.attributes = dict(attributes or {})
        verifier, judge = _OPDEFS[op_type]
        if not verifier(self):
            raise VerificationError('Operation of type "%s" failed verification.' % op_type)
        self.dtype, shape = judge(self)
        self.shape = tuple(int(s) for s in shape)
        self._id = None          # id inside the device graph once registered
        self._host = None        # initial value of a variable/constant before registration

    # -- type helpers
    @property
    def volume(self):
        return _vol(self.shape)

    @property
    def rank(self):
        return len(self.shape)

    @property
    def elementType(self):
        return self.dtype

    # -- value of a variable / constant
    @property
    def value(self):
        if self.opType not in ("variable", "constant"):
            return None
        if self._id is None:
            return self._host.copy()
        ptr, nbytes = self.device_ptr()
        out = np.empty(self.shape, self.dtype)
        capi.check(_lib().dopt_hip_copy_d2h(out.ctypes.data, ptr, nbytes))
        return out

    def set_value(self, array):
        a = np.ascontiguousarray(array, dtype=self.dtype).reshape(self.shape)
        if self._id is None:
            self._host = a.copy()
        else:
            ptr, nbytes = self.device_ptr()
            capi.check(_lib().dopt_hip_copy_h2d(ptr, a.ctypes.data, nbytes))

    def device_ptr(self):
        _register([self])
        p, n = C.c_void_p(), C.c_size_t()
        capi.check(_lib().dopt_hip_graph_value(_graph.get(), self._id, C.byref(p), C.byref(n)))
        return p.value or 0, n.value

    # -- operator sugar with the reference's scalar broadcasting (ops/package.d:94-168)
    def _binary(self, name, rhs):
        if isinstance(rhs, (int, np.integer)) and not isinstance(rhs, bool):
            rhs = int32Constant([], [int(rhs)])
        elif isinstance(rhs, (float, np.floating)):
            rhs = float32Constant([], [float(rhs)])
        if rhs.rank == 0 and self.rank != 0:
            return self._binary(name, repeat(rhs, self.volume).reshape(self.shape))
        if self.rank == 0 and rhs.rank != 0:
            return repeat(self, rhs.volume).reshape(rhs.shape)._binary(name, rhs)
        return Operation(name, [self, rhs])

    def __add__(self, rhs):
        return self._binary("add", rhs)

    def __sub__(self, rhs):
        return self._binary("sub", rhs)

    def __mul__(self, rhs):
        return self._binary("mul", rhs)

    def __truediv__(self, rhs):
        return self._binary("div", rhs)

    # opBinaryRight: '*' and '+' commute into opBinary; '-' and '/' put the constant on the left
    def __radd__(self, lhs):
        return self._binary("add", lhs)

    def __rmul__(self, lhs):
        return self._binary("mul", lhs)

    def __rsub__(self, lhs):
        return float32Constant([], [float(lhs)])._binary("sub", self)

    def __rtruediv__(self, lhs):
        return float32Constant([], [float(lhs)])._binary("div", self)

    def __neg__(self):
        return neg(self)

    def reshape(self, shape):
        return reshape(self, shape)

    def __repr__(self):
        return "%s%s" % (self.opType, list(self.shape))

    __hash__ = object.__hash__

    def eq(self, other):
        return Operation("eq", [self, other])


def topological_sort(ops):
    """ops/package.d:284-311: depth-first, dependencies first, each operation once."""
    order, seen = [], set()
    for root in ops:
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


def _register(ops):
    """Registers the operations (and what they depend on) with the device graph."""
    lib = _lib()
    g = _graph.get()
    for op in topological_sort(ops):
        if op._id is not None:
            continue
        deps = (C.c_int * _bmax(len(op.deps), 1))(*[d._id for d in op.deps])
        oid = C.c_int()
        capi.check(lib.dopt_hip_graph_add_op(g, op.opType.encode(), _CODE[op.dtype], len(op.shape),
                                             capi.sizes(op.shape), len(op.deps), deps, C.byref(oid)))
        op._id = oid.value
        for key, val in op.attributes.items():
            if isinstance(val, float):
                capi.check(lib.dopt_hip_graph_set_attr_double(g, op._id, key.encode(), val))
            elif isinstance(val, (int, np.integer)):
                capi.check(lib.dopt_hip_graph_set_attr_sizes(g, op._id, key.encode(), capi.sizes([val]), 1))
            else:
                capi.check(lib.dopt_hip_graph_set_attr_sizes(g, op._id, key.encode(), capi.sizes(val), len(val)))
        if op.opType in ("variable", "constant") and op._host is not None:
            host, op._host = op._host, None
            if host.size:
                ptr, nbytes = op.device_ptr()
                capi.check(lib.dopt_hip_copy_h2d(ptr, host.ctypes.data, nbytes))


# ------------------------------------------------------------------------------- op definitions

def _same_type(a, b):
    return a.dtype == b.dtype and a.shape == b.shape


ARITH = ("add", "sub", "mul", "div")
COMP = ("lt", "lte", "gt", "gte", "eq", "neq")
BINFUNC = ("max", "min", "pow")
UNFUNC = ("neg", "abs", "sgn", "exp", "log", "sqrt", "sin", "cos", "tan", "asin", "acos", "atan", "atan2", "sinh",
          "cosh", "tanh", "asinh", "acosh", "atanh")   # ops/math.d:71-76 (atan2 is listed as unary there)

for _n in ARITH + COMP + BINFUNC:   # ops/math.d:20-33
    register_operation(_n, lambda op: len(op.deps) == 2 and _same_type(op.deps[0], op.deps[1]),
                       lambda op: (op.deps[0].dtype, op.deps[0].shape))
for _n in UNFUNC:                   # ops/math.d:35-48
    register_operation(_n, lambda op: True, lambda op: (op.deps[0].dtype, op.deps[0].shape))


def _make_binary(name):
    def ctor(a, b):
        return Operation(name, [a, b])
    ctor.__name__ = name
    return ctor


def _make_unary(name):
    def ctor(a):
        return Operation(name, [a])
    ctor.__name__ = name
    return ctor


add, sub, mul, div = (_make_binary(n) for n in ARITH)
lt, lte, gt, gte, eq, neq = (_make_binary(n) for n in COMP)
max, min, pow = (_make_binary(n) for n in BINFUNC)   # noqa: A001 - reference op names
(neg, abs, sgn, exp, log, sqrt, sin, cos, tan, asin, acos, atan, _atan2_unary, sinh, cosh, tanh, asinh, acosh,   # noqa: A001
 atanh) = (_make_unary(n) for n in UNFUNC)

# ops/math.d:129-191
register_operation(
    "matmul",
    lambda op: (len(op.deps) == 2 and op.deps[0].rank == 2 and op.deps[1].rank == 2 and
                op.deps[0].dtype == op.deps[1].dtype and op.deps[0].shape[1] == op.deps[1].shape[0]),
    lambda op: (op.deps[0].dtype, (op.deps[0].shape[0], op.deps[1].shape[1])))


def _verify_sum(op):
    if len(op.deps) != 1 or "axes" not in op.attributes:
        return False
    axes = list(op.attributes["axes"])
    return all(a < op.deps[0].rank for a in axes) and len(set(axes)) == len(axes)


def _judge_sum(op):
    axes = op.attributes["axes"]
    return op.deps[0].dtype, tuple(s for i, s in enumerate(op.deps[0].shape) if i not in axes)


register_operation("sum", _verify_sum, _judge_sum)
register_operation("maxElement", _verify_sum, _judge_sum)
register_operation(
    "argmin",
    lambda op: len(op.deps) == 1 and "axis" in op.attributes and op.attributes["axis"] < op.deps[0].rank,
    lambda op: (int32_t, tuple(1 if i == op.attributes["axis"] else s for i, s in enumerate(op.deps[0].shape))))


def matmul(lhs, rhs):
    return Operation("matmul", [lhs, rhs])


def sum(op, axes=None):   # noqa: A001   ops/math.d:243-282
    if op.rank == 0:
        return op.reshape(op.shape)
    axes = list(range(op.rank)) if not axes else list(axes)
    # "Temporary speed enhancement: use BLAS to do row/col sums of matrices"
    if op.rank == 2 and len(axes) == 1:
        if axes[0] == 1:
            ones = float32Constant([op.shape[1], 1], np.ones(op.shape[1], np.float32))
            return matmul(op, ones).reshape([op.shape[0]])
        if axes[0] == 0:
            ones = float32Constant([1, op.shape[0]], np.ones(op.shape[0], np.float32))
            return matmul(ones, op).reshape([op.shape[1]])
        raise ValueError("axes[0] must be less than op.rank")
    return Operation("sum", [op], {"axes": axes})


def argmin(op, axis):
    return Operation("argmin", [op], {"axis": int(axis)})


def maxElement(op, axes=None):   # ops/math.d:345-359
    if op.rank == 0:
        return op.reshape(op.shape)
    axes = list(range(op.rank)) if not axes else list(axes)
    return Operation("maxElement", [op], {"axes": axes})


# ops/basic.d:29-170
def _verify_slice(op):
    if "start" not in op.attributes or "stop" not in op.attributes or len(op.deps) != 1:
        return False
    start, stop, shape = op.attributes["start"], op.attributes["stop"], op.deps[0].shape
    return (len(start) == len(stop) == len(shape) and all(a < s for a, s in zip(start, shape)) and
            all(b <= s for b, s in zip(stop, shape)) and all(a < b for a, b in zip(start, stop)))


register_operation("slice", _verify_slice,
                   lambda op: (op.deps[0].dtype,
                               tuple(b - a for a, b in zip(op.attributes["start"], op.attributes["stop"]))))
register_operation(
    "pad",
    lambda op: ("before" in op.attributes and "after" in op.attributes and len(op.deps) == 1 and
                len(op.attributes["before"]) == len(op.attributes["after"]) == op.deps[0].rank),
    lambda op: (op.deps[0].dtype, tuple(b + a + s for b, a, s in
                                        zip(op.attributes["before"], op.attributes["after"], op.deps[0].shape))))
register_operation(
    "reshape",
    lambda op: len(op.deps) == 1 and "shape" in op.attributes and _vol(op.attributes["shape"]) == op.deps[0].volume,
    lambda op: (op.deps[0].dtype, tuple(op.attributes["shape"])))
register_operation(
    "transpose",
    lambda op: (len(op.deps) == 1 and "order" in op.attributes and
                sorted(op.attributes["order"]) == list(range(op.deps[0].rank))),
    lambda op: (op.deps[0].dtype, tuple(op.deps[0].shape[i] for i in op.attributes["order"])))
register_operation(
    "repeat",
    lambda op: ("repetitions" in op.attributes and len(op.deps) == 1 and
                len(op.attributes["repetitions"]) == op.deps[0].rank and all(r > 0 for r in op.attributes["repetitions"])),
    lambda op: (op.deps[0].dtype, tuple(s * r for s, r in zip(op.deps[0].shape, op.attributes["repetitions"]))))
for _n in ("variable", "constant"):
    register_operation(_n, lambda op: len(op.deps) == 0 and "type" in op.attributes,
                       lambda op: op.attributes["type"])


register_operation("uniform", lambda op: len(op.deps) == 0 and "shape" in op.attributes,    # ops/random.d:19-37
                   lambda op: (float32_t, tuple(op.attributes["shape"])))


def uniformSample(shape):   # ops/random.d:48-51: fresh draws from (0, 1] at every evaluation
    return Operation("uniform", [], {"shape": [int(s) for s in shape]})


def slice(input, start, stop):   # noqa: A001, A002
    return Operation("slice", [input], {"start": list(start), "stop": list(stop)})


def pad(input, before, after):   # noqa: A002
    return Operation("pad", [input], {"before": list(before), "after": list(after)})


def reshape(input, shape):   # noqa: A002
    return Operation("reshape", [input], {"shape": [int(s) for s in shape]})


def transpose(input, order):   # noqa: A002
    return Operation("transpose", [input], {"order": list(order)})


def repeat(input, repetitions):   # noqa: A002
    """repeat(op, [r0, r1, ..]) tiles along each axis (ops/basic.d:318-331); repeat(op, n) adds a
    leading axis of n copies through a product with a ones vector (ops/basic.d:370-381)."""
    if isinstance(repetitions, (int, np.integer)):
        vec = input.reshape([1, input.volume])
        pattern = float32Constant([int(repetitions), 1], np.ones(int(repetitions), np.float32))
        return matmul(pattern, vec).reshape([int(repetitions)] + list(input.shape))
    if len(repetitions) != input.rank:
        raise ValueError("The length of repetitions must be the same as the rank of the input.")
    return Operation("repeat", [input], {"repetitions": list(repetitions)})


def _leaf(kind, dtype, shape, values):
    shape = tuple(int(s) for s in shape)
    dtype = np.dtype(dtype)
    op = Operation(kind, [], {"type": (dtype, shape)})
    del op.attributes["type"]   # not a payload a kernel reads
    if values is None:
        host = np.zeros(shape, dtype)
    else:
        host = np.asarray(values, dtype=dtype)
        if host.size != _vol(shape):
            raise ValueError("The length of defaultVal does not match type.volume.")
        host = host.reshape(shape).copy()
    op._host = host
    return op


def variable(dtype, shape, default=None):
    return _leaf("variable", dtype, shape, default)


def float32(shape=(), default=None):
    if isinstance(shape, (float, int)) and default is None:
        return _leaf("variable", np.float32, (), [float(shape)])
    return _leaf("variable", np.float32, shape, default)


def int32(shape=(), default=None):
    return _leaf("variable", np.int32, shape, default)


def constant(dtype, shape, values):
    return _leaf("constant", dtype, shape, values)


def float32Constant(shape, values=None):
    if isinstance(shape, (float, int)) and values is None:
        return _leaf("constant", np.float32, (), [float(shape)])
    return _leaf("constant", np.float32, shape, values)


def int32Constant(shape, values=None):
    if isinstance(shape, (int, np.integer)) and values is None:
        return _leaf("constant", np.int32, (), [int(shape)])
    return _leaf("constant", np.int32, shape, values)


# ops/nnet.d:42-236
def _conv_judge(op):
    x, w = op.deps
    pad_, st = op.attributes["padding"], op.attributes["stride"]
    return x.dtype, (x.shape[0], w.shape[0], (x.shape[2] + 2 * pad_[0] - w.shape[2]) // st[0] + 1,
                     (x.shape[3] + 2 * pad_[1] - w.shape[3]) // st[1] + 1)


register_operation(
    "convolution",
    lambda op: (len(op.deps) == 2 and op.deps[0].rank == 4 and op.deps[1].rank == 4 and
                op.deps[0].dtype == op.deps[1].dtype and op.deps[0].shape[1] == op.deps[1].shape[1]),
    _conv_judge)
register_operation(
    "maxpool",
    lambda op: len(op.deps) == 1 and op.deps[0].rank == 4 and len(op.attributes.get("dims", ())) == 2,
    lambda op: (op.deps[0].dtype, (op.deps[0].shape[0], op.deps[0].shape[1],
                                   op.deps[0].shape[2] // op.attributes["dims"][0],
                                   op.deps[0].shape[3] // op.attributes["dims"][1])))
register_operation("convolutionFeaturesGrad", lambda op: True,
                   lambda op: (op.deps[0].dtype, tuple(op.attributes["featuresShape"])))
register_operation("convolutionFiltersGrad", lambda op: True,
                   lambda op: (op.deps[0].dtype, tuple(op.attributes["filtersShape"])))
register_operation("maxpoolGrad", lambda op: True,
                   lambda op: (op.deps[0].dtype, tuple(op.attributes["featuresShape"])))
register_operation("softmax", lambda op: len(op.deps) == 1, lambda op: (op.deps[0].dtype, op.deps[0].shape))
register_operation("softmaxGrad", lambda op: len(op.deps) == 2, lambda op: (op.deps[1].dtype, op.deps[1].shape))
register_operation("relu", lambda op: len(op.deps) == 1, lambda op: (op.deps[0].dtype, op.deps[0].shape))
register_operation("reluGrad", lambda op: len(op.deps) == 3, lambda op: (op.deps[1].dtype, op.deps[1].shape))
register_operation("addBias", lambda op: True, lambda op: (op.deps[0].dtype, op.deps[0].shape))
register_operation("addBiasGrad", lambda op: True, lambda op: (op.deps[0].dtype, (op.deps[0].shape[1],)))
register_operation("batchNormTrain", lambda op: True,
                   lambda op: (op.deps[0].dtype, (op.deps[0].volume + 2 * op.deps[0].shape[1],)))
register_operation("batchNormGrad", lambda op: True,
                   lambda op: (op.deps[0].dtype, (op.deps[0].volume + op.deps[1].volume + op.deps[2].volume,)))
register_operation("batchNormInference", lambda op: True, lambda op: (op.deps[0].dtype, op.deps[0].shape))


def convolution(features, filters, padding=(0, 0), stride=(1, 1)):
    return Operation("convolution", [features, filters], {"padding": list(padding), "stride": list(stride)})


def convolutionTranspose(features, filters, padding=(0, 0), stride=(1, 1)):   # ops/nnet.d:305-315
    out = list(features.shape)
    for i in (0, 1):
        out[2 + i] = (out[2 + i] - 1) * stride[i] + filters.shape[2 + i] - 2 * padding[i]
    out[1] = filters.shape[1]
    return convolutionFeaturesGrad(features, filters, out, padding, stride)


def maxpool(features, dims):
    return Operation("maxpool", [features], {"dims": list(dims)})


def convolutionFeaturesGrad(parentGrad, filters, featuresShape, padding, stride):
    return Operation("convolutionFeaturesGrad", [parentGrad, filters],
                     {"featuresShape": list(featuresShape), "padding": list(padding), "stride": list(stride)})


def convolutionFiltersGrad(parentGrad, features, filtersShape, padding, stride):
    return Operation("convolutionFiltersGrad", [parentGrad, features],
                     {"filtersShape": list(filtersShape), "padding": list(padding), "stride": list(stride)})


def maxpoolGrad(parentGrad, op):
    return Operation("maxpoolGrad", [parentGrad, op, op.deps[0]],
                     {"featuresShape": list(op.deps[0].shape), "dims": list(op.attributes["dims"])})


def softmax(inputs):
    return Operation("softmax", [inputs])


def softmaxGrad(parentGrad, op):
    return Operation("softmaxGrad", [parentGrad, op])


def relu(inputs):
    return Operation("relu", [inputs])


def reluGrad(parentGrad, op):
    return Operation("reluGrad", [parentGrad, op, op.deps[0]])


def addBias(input, bias):   # noqa: A002
    return Operation("addBias", [input, bias])


def addBiasGrad(parentGrad):
    return Operation("addBiasGrad", [parentGrad])


def batchNormTrain(input, scale, bias, mean, var, momentum):   # noqa: A002   ops/nnet.d:476-489
    bnop = Operation("batchNormTrain", [input, scale, bias, mean, var], {"momentum": float(momentum)})
    v, c = input.volume, input.shape[1]
    return [slice(bnop, [0], [v]).reshape(input.shape), slice(bnop, [v], [v + c]), slice(bnop, [v + c], [v + 2 * c])]


def batchNormGrad(parentGrad, input, scale):   # noqa: A002
    return Operation("batchNormGrad", [parentGrad, input, scale])


def batchNormInference(input, scale, bias, mean, var):   # noqa: A002
    return Operation("batchNormInference", [input, scale, bias, mean, var])


# ------------------------------------------------------------------------------- gradients (grads/*.d)

def _reg_grads():
    g = register_gradient
    # grads/math.d
    g("matmul", lambda op, pg: [matmul(pg, transpose(op.deps[1], [1, 0])), matmul(transpose(op.deps[0], [1, 0]), pg)])

    def sum_grad(op, pg):
        if op.volume == 1:
            return [repeat(pg, op.deps[0].volume).reshape(op.deps[0].shape)]
        tmp_shape, reps = list(op.deps[0].shape), [1] * op.deps[0].rank
        for a in op.attributes["axes"]:
            reps[a] = tmp_shape[a]
            tmp_shape[a] = 1
        return [repeat(pg.reshape(tmp_shape), reps)]
    g("sum", sum_grad)
    g("add", lambda op, pg: [pg, pg])
    g("sub", lambda op, pg: [pg, neg(pg)])
    g("mul", lambda op, pg: [pg * op.deps[1], pg * op.deps[0]])
    g("div", lambda op, pg: [pg / op.deps[1], neg(pg * op.deps[0]) / (op.deps[1] * op.deps[1])])
    g("pow", lambda op, pg: [pg * op.deps[1] * pow(op.deps[0], op.deps[1] - 1), pg * op.deps[1] * log(op.deps[0])])
    g("min", lambda op, pg: [op.deps[0].eq(op) * pg, op.deps[1].eq(op) * pg])
    g("max", lambda op, pg: [op.deps[0].eq(op) * pg, op.deps[1].eq(op) * pg])
    g("neg", lambda op, pg: [neg(pg)])
    g("abs", lambda op, pg: [pg * sgn(op.deps[0])])
    g("exp", lambda op, pg: [pg * op])
    g("log", lambda op, pg: [pg / op.deps[0]])
    g("sqrt", lambda op, pg: [pg / op])
    # grads/basic.d
    g("transpose", lambda op, pg: [transpose(pg, [op.attributes["order"].index(i)
                                                  for i in range(len(op.attributes["order"]))])])
    g("slice", lambda op, pg: [pad(pg, op.attributes["start"],
                                   [s - e for s, e in zip(op.deps[0].shape, op.attributes["stop"])])])
    g("pad", lambda op, pg: [slice(pg, op.attributes["before"],
                                   [s + b for s, b in zip(op.deps[0].shape, op.attributes["before"])])])
    g("reshape", lambda op, pg: [pg.reshape(op.deps[0].shape)])

    def repeat_grad(op, pg):
        reps = op.attributes["repetitions"]
        tmp_shape = []
        for r, s in zip(reps, op.deps[0].shape):
            tmp_shape += [r, s]
        return [sum(pg.reshape(tmp_shape), list(range(0, len(tmp_shape), 2)))]
    g("repeat", repeat_grad)
    # grads/nnet.d
    g("convolution", lambda op, pg: [
        convolutionFeaturesGrad(pg, op.deps[1], op.deps[0].shape, op.attributes["padding"], op.attributes["stride"]),
        convolutionFiltersGrad(pg, op.deps[0], op.deps[1].shape, op.attributes["padding"], op.attributes["stride"])])
    g("convolutionFeaturesGrad", lambda op, pg: [
        convolution(pg, op.deps[1], op.attributes["padding"], op.attributes["stride"]),
        convolutionFiltersGrad(op.deps[0], pg, op.deps[1].shape, op.attributes["padding"], op.attributes["stride"])])
    g("maxpool", lambda op, pg: [maxpoolGrad(pg, op)])
    g("softmax", lambda op, pg: [softmaxGrad(pg, op)])
    g("relu", lambda op, pg: [reluGrad(pg, op)])
    g("addBias", lambda op, pg: [pg, addBiasGrad(pg)])

    def bn_grad(op, pg):
        x, scale, bias = op.deps[0], op.deps[1], op.deps[2]
        trimmed = slice(pg, [0], [x.volume]).reshape(x.shape)
        packed = batchNormGrad(trimmed, x, scale)
        packed = packed.reshape([packed.volume])
        v0, v1, v2 = x.volume, scale.volume, bias.volume
        return [slice(packed, [0], [v0]).reshape(x.shape),
                slice(packed, [v0], [v0 + v1]).reshape(scale.shape),
                slice(packed, [v0 + v1], [v0 + v1 + v2]).reshape(bias.shape),
                float32(op.deps[3].shape), float32(op.deps[4].shape)]
    g("batchNormTrain", bn_grad)


_reg_grads()


def grad(objective, wrt):
    """Reverse-mode automatic differentiation (grads/package.d:39-110)."""
    if objective.volume != 1:
        raise ValueError("The objective must have a volume of one")
    if objective.dtype != float32_t:
        raise ValueError("The objective must have a floating point type")
    ops = topological_sort([objective])
    grads = {id(objective): float32(objective.shape, [1.0])}
    for op in reversed(ops):
        fn = _GRADS.get(op.opType)
        op_grad = grads.get(id(op))
        if fn is None or op_grad is None:
            continue
        for d, g in zip(op.deps, fn(op, op_grad)):
            cur = grads.get(id(d))
            grads[id(d)] = g if cur is None else cur + g
    for i, w in enumerate(wrt):
        if id(w) not in grads:
            raise ValueError("Could not find wrt[%d] in the operation graph" % i)
    return [grads[id(w)] for w in wrt]


# ------------------------------------------------------------------------------- evaluation

PLAN_VIEWS = 1
PLAN_TIMING = 2
PLAN_FUSE = 4
PLAN_OVERLAP = 8
PLAN_GRAPH = 16
PLAN_OVERLAP_LIGHT = 32
PLAN_TIMING_SHAPES = 64


class Plan:
    """class CUDAPlan (cuda/package.d:261-433) for this backend: HIPPlan behind the C ABI."""

    def __init__(self, outputs, flags=0):
        self.outputs = list(outputs)
        _register(self.outputs)
        ids = (C.c_int * _bmax(len(self.outputs), 1))(*[o._id for o in self.outputs])
        h = C.c_void_p()
        capi.check(_lib().dopt_hip_plan_create(_graph.get(), len(self.outputs), ids, flags, C.byref(h)))
        self._h = h

    def execute(self, args=None, rets=None):
        """args: {variable Operation: numpy array (host) | ops.Tensor | int device pointer}.
        rets: optional list of device pointers (ints) / Tensors / None, one per output; when omitted,
        fresh host arrays are returned (Plan.execute(args) of core/package.d:158-170)."""
        lib = _lib()
        args = args or {}
        n = len(args)
        ids = (C.c_int * _bmax(n, 1))()
        ptrs = (C.c_void_p * _bmax(n, 1))()
        on_host = (C.c_int * _bmax(n, 1))()
        keep = []
        for i, (var, val) in enumerate(args.items()):
            _register([var])
            ids[i] = var._id
            if isinstance(val, np.ndarray) or np.isscalar(val) or isinstance(val, (list, tuple)):
                a = np.ascontiguousarray(val, dtype=var.dtype)
                if a.size != var.volume:
                    raise capi.HipError(1, "Mismatch in buffer size")
                keep.append(a)
                ptrs[i] = a.ctypes.data
                on_host[i] = 1
            else:
                ptrs[i] = val.ptr if hasattr(val, "ptr") else int(val)
                on_host[i] = 0
        if rets is not None:
            rp = (C.c_void_p * _bmax(len(rets), 1))()
            for i, r in enumerate(rets):
                rp[i] = None if r is None else (r.ptr if hasattr(r, "ptr") else int(r))
            capi.check(lib.dopt_hip_plan_execute(self._h, n, ids, ptrs, on_host, len(rets), rp))
            return None
        capi.check(lib.dopt_hip_plan_execute(self._h, n, ids, ptrs, on_host, 0, None))
        return [self.result(o) for o in self.outputs]

    def result_ptr(self, op):
        p, nbytes = C.c_void_p(), C.c_size_t()
        capi.check(_lib().dopt_hip_plan_result(self._h, op._id, C.byref(p), C.byref(nbytes)))
        return p.value or 0, nbytes.value

    def result(self, op):
        ptr, nbytes = self.result_ptr(op)
        out = np.empty(op.shape, op.dtype)
        capi.check(_lib().dopt_hip_copy_d2h(out.ctypes.data, ptr, nbytes))
        return out

    def stats(self):
        k, b = C.c_size_t(), C.c_size_t()
        capi.check(_lib().dopt_hip_plan_stats(self._h, C.byref(k), C.byref(b)))
        return {"kernels": k.value, "buffer_bytes": b.value}

    def recordings(self):
        a, b = C.c_size_t(), C.c_size_t()
        capi.check(_lib().dopt_hip_plan_recordings(self._h, C.byref(a), C.byref(b)))
        return {"recorded": a.value, "replays": b.value}

    def profile(self):
        need = C.c_size_t()
        capi.check(_lib().dopt_hip_plan_profile(self._h, None, 0, C.byref(need)))
        buf = C.create_string_buffer(need.value)
        capi.check(_lib().dopt_hip_plan_profile(self._h, buf, need.value, None))
        out = {}
        for line in buf.value.decode().splitlines():
            name, usec, count = line.split()
            out[name] = (float(usec), int(count))
        return out

    def cleanup(self):
        if self._h:
            _lib().dopt_hip_plan_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.cleanup()
        except Exception:
            pass


def compile(outputs, flags=0):   # noqa: A001   core/package.d:141-156
    return Plan(outputs, flags)


def evaluate(ops, args=None):
    """evaluateCUDA (cuda/package.d:448-470): one-off plan, results as host arrays."""
    single = isinstance(ops, Operation)
    plan = Plan([ops] if single else list(ops))
    try:
        res = plan.execute(args)
    finally:
        plan.cleanup()
    return res[0] if single else res


def list_operations():
    need = C.c_size_t()
    capi.check(_lib().dopt_hip_list_operations(None, 0, C.byref(need)))
    buf = C.create_string_buffer(need.value)
    capi.check(_lib().dopt_hip_list_operations(buf, need.value, None))
    return buf.value.decode().split()
