"""Builds the HIP search core (libvsag_amd.so) and the host C++ layer for gfx950 with hipcc.

Run as `python -m vsag_amd.build`; `__graft_entry__.build()` calls `build_all()`.  hipcc cross-compiles
without a GPU.  Objects go to vsag_amd/lib/obj, libraries to vsag_amd/lib.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

ROOT = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(ROOT, "csrc")
HOST = os.path.join(ROOT, "host")
LIB = os.path.join(ROOT, "lib")
OBJ = os.path.join(LIB, "obj")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden",
    # packed fp32 VALU forms are switched off on purpose for this machine pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-attributes",
]
KERNEL_SOURCES = ["runtime.hip", "store.hip", "quantize.hip", "prepare.hip", "scan.hip", "prefilter.hip", "prefilter_i8.hip", "prefilter_rb.hip", "prefilter_h16.hip", "ivf.hip", "ivf_i8.hip", "ivf_pq.hip",
                  "kmeans.hip", "lookup.hip", "export.hip", "scan_one.hip", "pq.hip"]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip())
    if proc.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_kernels(verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    sources = [s for s in KERNEL_SOURCES if os.path.exists(os.path.join(CSRC, s))]

    def compile_one(src):
        obj = os.path.join(OBJ, src.replace(".hip", ".o"))
        out = _run([HIPCC] + HIP_FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj])
        if verbose and out:
            print(out)
        return obj

    with ThreadPoolExecutor(max_workers=6) as pool:
        objs = list(pool.map(compile_one, sources))
    lib = os.path.join(LIB, "libvsag_amd.so")
    _run([HIPCC, "-shared", "-fPIC", "--offload-arch=gfx950", "-o", lib] + objs)
    if verbose:
        print("built", lib)
    return lib


def build_host(verbose=True):
    if not os.path.isdir(HOST):
        return None
    sources = sorted(f for f in os.listdir(HOST) if f.endswith(".cpp"))
    if not sources:
        return None
    lib = os.path.join(LIB, "libvsag_amd_host.so")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-fvisibility=hidden",
           "-I" + os.path.join(ROOT, "..", "include"),
           "-o", lib] + [os.path.join(HOST, s) for s in sources] + [
               "-L" + LIB, "-lvsag_amd", "-Wl,-rpath,$ORIGIN", "-lpthread"]
    out = _run(cmd)
    if verbose:
        if out:
            print(out)
        print("built", lib)
    return lib


def build_host_example(verbose=True):
    """tests/cpp/host_api.cpp: a C++ program against vsag_host.h, run by the tests (it must be built before them)."""
    src = os.path.join(ROOT, "..", "tests", "cpp", "host_api.cpp")
    if not os.path.exists(src):
        return None
    exe = os.path.join(LIB, "host_api_test")
    out = _run(["g++", "-O2", "-std=c++17", "-Wall", "-I" + HOST, "-o", exe, src, "-L" + LIB, "-lvsag_amd_host",
                "-lvsag_amd", "-Wl,-rpath,$ORIGIN", "-lpthread"])
    if verbose:
        if out:
            print(out)
        print("built", exe)
    return exe


def build_all(verbose=True):
    build_kernels(verbose)
    build_host(verbose)
    build_host_example(verbose)


if __name__ == "__main__":
    build_all()
    sys.exit(0)
