"""Builds libmni_rocm.so (HIP kernels + C ABI) for gfx950 with hipcc.

Usage: python -m framework_amd.build [--force]

The library is built in-tree (framework_amd/lib/libmni_rocm.so).  hipcc
cross-compiles gfx950 code objects without a GPU, so this runs anywhere the
ROCm toolchain is installed.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "lib", "obj")
LIB = os.path.join(HERE, "lib", "libmni_rocm.so")
SOURCES = ["device.hip", "gemm_mfma.hip", "gemm_direct.hip", "gemm_panel.hip", "gemm_tiny.hip", "gemm_fewrows.hip", "gemm_outer.hip", "gemm_skinny.hip", "gemm_gemv.hip", "gemm_fewrows_nt.hip", "gemm.hip", "elementwise.hip", "yardstick.hip", "attention.hip", "sequence.hip", "engine.hip"]
HEADERS = ["common.h", "gemm_internal.h", os.path.join("..", "..", "include", "mni_rocm.h")]

# -packed-fp32-ops is switched off for device code: hipcc must not form
# v_pk_*_f32 from ordinary float arithmetic on this target.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc():
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "not a recognized feature for this target" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    hipcc = _hipcc()
    headers = [os.path.normpath(os.path.join(CSRC, h)) for h in HEADERS]
    jobs = []
    objs = []
    for src in SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ, src.replace(".hip", ".o"))
        objs.append(o)
        if force or _stale(o, [s] + headers):
            jobs.append([hipcc] + FLAGS + ["-c", s, "-o", o])
    with ThreadPoolExecutor(max_workers=min(6, os.cpu_count() or 1)) as ex:
        for out in ex.map(_run, jobs):
            if verbose and out.strip():
                print(out)
    if force or jobs or _stale(LIB, objs):
        out = _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
        if verbose and out.strip():
            print(out)
    if verbose:
        print("built %s (%d translation units recompiled)" % (LIB, len(jobs)))
    build_node_addon(force or bool(jobs), verbose)
    build_step_bench(force or bool(jobs), verbose)
    return LIB


STEP_BENCH = os.path.join(HERE, "lib", "mlp_step_bench")


def build_step_bench(force=False, verbose=True):
    """The README training step driven through the engine-level C ABI from plain C (csrc/mlp_step_bench.c): what a
    step costs without a language binding in the loop.  bench.py runs it beside its own (ctypes) figure."""
    src = os.path.join(CSRC, "mlp_step_bench.c")
    inc = os.path.normpath(os.path.join(CSRC, "..", "..", "include"))
    if force or _stale(STEP_BENCH, [src, LIB, os.path.join(inc, "mni_rocm.h")]):
        _run(["gcc", "-O2", "-std=c11", "-D_POSIX_C_SOURCE=199309L", "-Wall", "-I" + inc, src, "-o", STEP_BENCH, "-L" + os.path.dirname(LIB), "-lmni_rocm",
              "-Wl,-rpath,$ORIGIN"])
        if verbose:
            print("built %s" % STEP_BENCH)
    return STEP_BENCH


NODE_ADDON = os.path.join(HERE, "lib", "mni_rocm.node")
NODE_INCLUDE = "/usr/include/node"


def build_node_addon(force=False, verbose=True):
    """The Node-API shim (csrc/napi_shim.cpp) over the engine-level ABI.  Needs
    only g++ and node_api.h; skipped where the Node headers are not installed."""
    src = os.path.join(CSRC, "napi_shim.cpp")
    if not os.path.exists(os.path.join(NODE_INCLUDE, "node_api.h")):
        if verbose:
            print("node_api.h not found: Node addon not built")
        return None
    if force or _stale(NODE_ADDON, [src, LIB, os.path.normpath(os.path.join(CSRC, HEADERS[2]))]):
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-I" + NODE_INCLUDE, src, "-o", NODE_ADDON,
              "-L" + os.path.dirname(LIB), "-lmni_rocm", "-Wl,-rpath,$ORIGIN"])
        if verbose:
            print("built %s" % NODE_ADDON)
    return NODE_ADDON


if __name__ == "__main__":
    build(force="--force" in sys.argv)
