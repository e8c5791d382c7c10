"""Builds libstaf_hip.so (the C-ABI library with the gfx950 kernels) in-tree with hipcc.

    python -m alphanesgpu_amd.build [--force]

hipcc cross-compiles for gfx950 without a GPU.  The library lands in
alphanesgpu_amd/lib/libstaf_hip.so, next to the sources it is built from.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libstaf_hip.so")
SOURCES = ["staf_runtime.hip", "staf_desc.hip", "staf_af.hip", "staf_force.hip", "staf_api.hip", "staf_mlp_dev.hip", "staf_mlp.cpp"]
HEADERS = ["staf_common.hpp", "staf_tile.hpp", "staf_reduce.hpp", "staf_tri.hpp", "staf_force3.hpp", "staf_transpose.hpp", "staf_mlp_dev.hpp", "staf_mlp_internal.h", os.path.join("..", "..", "include", "staf_ops.h"),
           os.path.join("..", "..", "include", "staf.h"), os.path.join("..", "..", "include", "staf_mlp.h")]
ARCH = "gfx950"
# packed-fp32 instructions are switched off for all device code
HIPCC_FLAGS = ["-O3", "-std=c++17", "-fPIC", f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang",
               "-packed-fp32-ops", "-Wno-unused-result"]


def _hipcc():
    for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if c and (os.path.isabs(c) and os.path.exists(c) or not os.path.isabs(c)):
            return c
    return "hipcc"


def _stale(target, deps):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(d) > t for d in deps)


def build(force=False, verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    objdir = os.path.join(LIBDIR, "obj")
    os.makedirs(objdir, exist_ok=True)
    hdrs = [os.path.join(CSRC, h) for h in HEADERS]
    jobs = []
    objs = []
    for s in SOURCES:
        src = os.path.join(CSRC, s)
        obj = os.path.join(objdir, os.path.splitext(s)[0] + ".o")
        objs.append(obj)
        if force or _stale(obj, [src] + hdrs):
            jobs.append([_hipcc()] + HIPCC_FLAGS + ["-c", src, "-o", obj])

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in r.stdout.splitlines() if "not a recognized feature" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed:\n{out}")
        if verbose and out.strip():
            print(out)

    with ThreadPoolExecutor(max_workers=4) as ex:
        list(ex.map(run, jobs))
    if force or jobs or _stale(LIB, objs):
        run([_hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB] + objs)
    return LIB


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
