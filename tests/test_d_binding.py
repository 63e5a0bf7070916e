"""The D package under hip/ cannot be compiled here (no D compiler), so what can be checked mechanically is:
its extern(C) declarations are exactly what the C headers give, every declared function is exported by the
built library, every call the D modules make into the library matches a declaration (name and argument count),
and the operations the D registry names are the operations the library's own planner has kernels for."""
import ctypes as C
import importlib.util
import os
import re

from dopt_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIP = os.path.join(ROOT, "hip")
SRC = os.path.join(HIP, "source", "dopt", "hip")


def _gen():
    spec = importlib.util.spec_from_file_location("gen_shim", os.path.join(HIP, "gen_shim.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _declared():
    """name -> number of parameters, from shim.d."""
    text = open(os.path.join(SRC, "shim.d")).read()
    out = {}
    for m in re.finditer(r"^[\w\(\)\* ]+?\b(dopt_hip_\w+)\((.*)\);$", text, flags=re.M):
        params = m.group(2).strip()
        out[m.group(1)] = 0 if not params else _top_level_commas(params) + 1
    return out


def _top_level_commas(s):
    depth = n = 0
    for ch in s:
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        elif ch == "," and depth == 0:
            n += 1
    return n


def _calls(text):
    """(name, argument count) of every call of a library function in D source text."""
    out = []
    for m in re.finditer(r"\b(dopt_hip_\w+)\s*\(", text):
        i, depth = m.end(), 1
        while depth:
            depth += {"(": 1, ")": -1}.get(text[i], 0)
            i += 1
        args = text[m.end():i - 1].strip()
        out.append((m.group(1), 0 if not args else _top_level_commas(args) + 1))
    return out


def test_shim_is_what_the_headers_give():
    gen = _gen()
    assert open(os.path.join(SRC, "shim.d")).read() == gen.render()


def test_every_declared_function_is_exported_by_the_library():
    declared = _declared()
    assert len(declared) >= 90
    assert set(declared) == set(capi.exported_symbols()) | {
        n for n in declared if n.startswith(("dopt_hip_graph_", "dopt_hip_plan_", "dopt_hip_register_", "dopt_hip_deregister_",
                                             "dopt_hip_list_"))}
    lib = C.CDLL(capi.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name


def test_every_call_from_d_matches_a_declaration():
    declared = _declared()
    seen = set()
    for fn in sorted(os.listdir(SRC)):
        if fn == "shim.d" or not fn.endswith(".d"):
            continue
        text = re.sub(r"//.*", "", open(os.path.join(SRC, fn)).read())
        text = re.sub(r"/\*\*.*?\*/", "", text, flags=re.S)
        structs = set(re.findall(r"^struct (\w+)$", open(os.path.join(SRC, "shim.d")).read(), flags=re.M))
        for name, nargs in _calls(text):
            if name in structs:      # a struct literal, not a call
                continue
            assert name in declared, "%s calls %s, which shim.d does not declare" % (fn, name)
            assert nargs == declared[name], "%s calls %s with %d arguments, declared with %d" % (fn, name, nargs, declared[name])
            seen.add(name)
    # the kernel entry points of every reference operation are reached from D
    for must in ("dopt_hip_pointwise", "dopt_hip_reduce", "dopt_hip_argmin", "dopt_hip_slice", "dopt_hip_pad", "dopt_hip_repeat",
                 "dopt_hip_transpose2d", "dopt_hip_sgemm", "dopt_hip_conv_fwd", "dopt_hip_conv_bwd_data", "dopt_hip_conv_bwd_filter",
                 "dopt_hip_maxpool_fwd", "dopt_hip_maxpool_bwd", "dopt_hip_softmax_fwd", "dopt_hip_softmax_bwd", "dopt_hip_relu_fwd",
                 "dopt_hip_relu_bwd", "dopt_hip_bias_fwd", "dopt_hip_bias_bwd", "dopt_hip_bn_train", "dopt_hip_bn_grad",
                 "dopt_hip_bn_infer", "dopt_hip_uniform", "dopt_hip_sgd_step", "dopt_hip_adam_step", "dopt_hip_amsgrad_step",
                 "dopt_hip_plan_create", "dopt_hip_plan_execute", "dopt_hip_graph_add_op", "dopt_hip_register_kernel"):
        assert must in seen, must


def test_d_registry_names_the_operations_the_library_has_kernels_for():
    names = set()
    for fn in ("basic.d", "math.d", "nnet.d", "random.d"):
        text = open(os.path.join(SRC, fn)).read()
        names |= set(re.findall(r'registerHIPKernel\("(\w+)"', text))
        for arr in re.findall(r"string\[\] \w+ = \[(.*?)\];", text, flags=re.S):
            names |= set(re.findall(r'"(\w+)"', arr))
    lib = capi.load()
    lib.dopt_hip_list_operations.argtypes = [C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]
    need = C.c_size_t()
    assert lib.dopt_hip_list_operations(None, 0, C.byref(need)) == 0
    buf = C.create_string_buffer(need.value)
    assert lib.dopt_hip_list_operations(buf, need.value, None) == 0
    native = set(buf.value.decode().split()) - {"variable", "reshape", "constant"}
    assert names == native, (sorted(names - native), sorted(native - names))


def test_dub_package_mirrors_the_reference_layout():
    import json
    d = json.load(open(os.path.join(HIP, "dub.json")))
    assert d["name"] == "hip" and {"dopt:core", "dopt:cpu"} <= set(d["dependencies"]) and "dopthip" in d["libs"]
    patch = open(os.path.join(HIP, "integration.patch")).read()
    assert '"hip"' in patch and "version(Have_dopt_hip)" in patch and "import dopt.hip;" in patch
    for fn in ("shim.d", "package.d", "basic.d", "math.d", "nnet.d", "random.d", "online.d"):
        text = open(os.path.join(SRC, fn)).read()
        code = re.sub(r"/\*\*.*?\*/", "", re.sub(r"//.*", "", text), flags=re.S)
        assert code.count("{") == code.count("}") and code.count("(") == code.count(")") and \
            code.count("[") == code.count("]"), fn
        assert re.search(r"^module dopt\.hip(\.\w+)?;$", text, flags=re.M), fn
