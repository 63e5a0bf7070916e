"""Builds dopt_amd/libdopthip.so from dopt_amd/csrc with hipcc for gfx950.

Usage: python -m dopt_amd.build [--force]
The library is built in-tree (next to this file) so that it travels with the source tree.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_PATH = os.path.join(HERE, "libdopthip.so")

SOURCES = ["runtime.cpp", "rtc_ops.cpp", "layout.hip", "nn.hip", "bn.hip", "optim.hip", "sgemm.hip", "conv.hip", "conv_smallc.hip", "tiny.hip",
           "plan.cpp"]
HEADERS = ["common.h", "mfma_core.h", "pool2x2.h", "pw_ops.h", "plan.h", os.path.join("..", "..", "include", "dopt_hip.h"),
           os.path.join("..", "..", "include", "dopt_hip_plan.h")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
# -ffp-contract=off: fused kernels must round once per node of the op graph they replace.
# -fhip-fp32-correctly-rounded-divide-sqrt: '/' and sqrtf are IEEE, as on the CPU evaluator.
# packed fp32 VALU ops are disabled library-wide.
FLAGS = ["--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-x", "hip", "-ffp-contract=off",
         "-fhip-fp32-correctly-rounded-divide-sqrt", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
         "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes"]


def _newer(target, deps):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.exists(d) and os.path.getmtime(d) <= t for d in deps)


def _compile(src, force):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    deps = [os.path.join(CSRC, src)] + [os.path.join(CSRC, h) for h in HEADERS]
    deps = [d for d in deps if os.path.exists(d)]
    if not force and _newer(obj, deps):
        return obj, None
    cmd = [HIPCC] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, res.stdout, res.stderr))
    return obj, res.stderr


def build(force=False, verbose=False):
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(sources))) as ex:
        results = list(ex.map(lambda s: _compile(s, force), sources))
    objs = [o for o, _ in results]
    if verbose:
        for (_, log), s in zip(results, sources):
            if log and "warning" in log and "packed-fp32-ops" not in log:
                sys.stderr.write("[%s]\n%s\n" % (s, log))
    if force or not _newer(LIB_PATH, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs + \
              ["-L/opt/rocm/lib", "-lhiprtc", "-Wl,-rpath,/opt/rocm/lib"]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError("link failed:\n%s\n%s" % (res.stdout, res.stderr))
    return LIB_PATH


if __name__ == "__main__":
    print(build(force="--force" in sys.argv, verbose=True))
