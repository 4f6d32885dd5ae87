"""Compiles libmcsparse.so (host C++ + HIP kernels for gfx950) in-tree with hipcc.

Every source is compiled to an object of its own (in parallel), then linked with a version script
that exports the `mcsparse*` C functions and nothing else, under the SONAME libmcsparse.so.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libmcsparse.so")
EXPORTS = os.path.join(CSRC, "exports.map")

SOURCES = ["api_helper.cpp", "api_compute.cpp", "api_legacy.cpp", "api_sort.cpp", "topology.cpp", "analysis.hip", "spmv.hip",
           "spmv_banded.hip", "spmm.hip", "spmm_blocks.hip", "spmm_strips.hip", "spmm_long.hip", "convert.hip", "static_scratch.hip"]
HEADERS = ["internal.h", "device_util.h", "spmm_device.h"]

COMPILE_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-Wall",
    # compiler-generated packed fp32 math is switched off for every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]
LINK_FLAGS = ["--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-soname,libmcsparse.so",
              "-Wl,--version-script=" + EXPORTS]


def _run(cmd):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise subprocess.CalledProcessError(proc.returncode, cmd, output=out)
    return out


def _stale(obj, deps):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    return any(os.path.getmtime(d) > t for d in deps)


def build_library(verbose=False, incremental=False, jobs=None):
    """Runs hipcc; raises CalledProcessError with the compiler output on failure.

    incremental=True recompiles only the sources that changed since their object was written (for
    work on one kernel file); the default compiles everything.
    """
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    common = [os.path.join(CSRC, h) for h in HEADERS] + [os.path.join(INCLUDE, "mcsparse.h")]
    todo = []
    objects = []
    for s in SOURCES:
        src = os.path.join(CSRC, s)
        obj = os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o")
        objects.append(obj)
        if not incremental or _stale(obj, [src] + common):
            todo.append([hipcc] + COMPILE_FLAGS + ["-I", INCLUDE, "-c", src, "-o", obj])
    jobs = jobs or min(8, os.cpu_count() or 1)
    try:
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            outs = list(pool.map(_run, todo))
        outs.append(_run([hipcc] + LINK_FLAGS + ["-o", LIB_PATH] + objects))
    except subprocess.CalledProcessError as e:
        if verbose:
            print(e.output)
        raise
    if verbose:
        text = "\n".join(o for o in outs if o.strip())
        if text:
            print(text)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True, incremental="--incremental" in sys.argv))
