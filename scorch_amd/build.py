"""Compiles scorch_amd/csrc/*.hip into scorch_amd/libscorch_hip.so for gfx950.

    python -m scorch_amd.build [--force]

hipcc cross-compiles without a GPU, so this runs on any host that has ROCm.
The library is kept in-tree, next to this file.
"""
from __future__ import annotations

import glob
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libscorch_hip.so")
OBJ_DIR = os.path.join(SRC_DIR, "obj")  # one object per source, rebuilt only when stale

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC",
    # packed fp32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results stay in ordinary vector registers: the attention kernel feeds them
    # straight to vector instructions, and accumulator registers would cost copies
    "-mllvm", "-amdgpu-mfma-vgpr-form",
    # floating-point atomic adds (SpGEMM accumulators) as the hardware's add instructions, not
    # compare-and-swap loops; their targets are LDS and ordinary device memory
    "-munsafe-fp-atomics",
    # (an unroll request the optimizer declines, e.g. in a loop it has already restructured, is no news)
    "-fvisibility=hidden", "-Wall", "-Wno-unused-function", "-Wno-pass-failed",
]


def sources():
    return sorted(glob.glob(os.path.join(SRC_DIR, "*.hip")))


def _headers():
    return glob.glob(os.path.join(SRC_DIR, "*.hpp")) + glob.glob(
        os.path.join(os.path.dirname(PKG_DIR), "include", "*.h"))


def _newer(target, deps) -> bool:
    """True if `target` is missing or older than any of `deps`."""
    if not os.path.exists(target):
        return True
    built = os.path.getmtime(target)
    return any(os.path.getmtime(d) > built for d in deps)


def _run_hipcc(args, verbose):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found: cannot build libscorch_hip.so")
    cmd = [hipcc] + list(args)
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature name and says so: harmless
    noise = [l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + "\n".join(noise))
    if verbose and noise:
        print("\n".join(noise), flush=True)


def _object_of(src) -> str:
    return os.path.join(OBJ_DIR, os.path.splitext(os.path.basename(src))[0] + ".o")


def _compile(src, verbose):
    obj = _object_of(src)
    tmp = obj + ".tmp"
    _run_hipcc(HIPCC_FLAGS + ["-c", src, "-o", tmp], verbose)
    os.replace(tmp, obj)
    return obj


def build_library(force: bool = False, verbose: bool = False) -> str:
    """Build libscorch_hip.so: every source that is newer than its object (all of
    them when ``force``) is compiled, the sources side by side, and the objects
    are linked.  Returns the library path."""
    srcs = sources()
    headers = _headers()
    os.makedirs(OBJ_DIR, exist_ok=True)
    todo = [s for s in srcs if force or _newer(_object_of(s), [s] + headers)]
    if todo:
        with ThreadPoolExecutor(max_workers=min(len(todo), os.cpu_count() or 1)) as pool:
            list(pool.map(lambda s: _compile(s, verbose), todo))
    objs = [_object_of(s) for s in srcs]
    if todo or _newer(LIB_PATH, objs):
        tmp = LIB_PATH + ".tmp"
        _run_hipcc(["-shared", "-fPIC", "--offload-arch=gfx950", "-fvisibility=hidden"] + objs + ["-o", tmp], verbose)
        os.replace(tmp, LIB_PATH)
    return LIB_PATH


HOST_DEMO_SRC = os.path.join(os.path.dirname(PKG_DIR), "tests", "host_c", "plan_demo.c")
HOST_DEMO_BIN = os.path.join(os.path.dirname(PKG_DIR), "tests", "host_c", "plan_demo")


def build_host_demo(verbose: bool = False) -> str:
    """Compile tests/host_c/plan_demo.c, a plain C99 host of the library (the C ABI and the HIP
    runtime, nothing else), with gcc.  Returns the program's path.  Needs no GPU to build."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    gcc = shutil.which("gcc")
    if not gcc:
        raise RuntimeError("gcc not found: cannot build the C host demo")
    cmd = [gcc, "-std=c99", "-Wall", "-Werror", "-O1", "-D__HIP_PLATFORM_AMD__",
           "-I", os.path.join(os.path.dirname(PKG_DIR), "include"), "-I", os.path.join(rocm, "include"),
           HOST_DEMO_SRC, "-L", PKG_DIR, "-l:libscorch_hip.so", "-L", os.path.join(rocm, "lib"), "-lamdhip64", "-lm",
           "-Wl,-rpath,$ORIGIN/../../scorch_amd", "-Wl,-rpath," + os.path.join(rocm, "lib"), "-o", HOST_DEMO_BIN + ".tmp"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("gcc failed:\n" + proc.stdout)
    os.replace(HOST_DEMO_BIN + ".tmp", HOST_DEMO_BIN)
    return HOST_DEMO_BIN


if __name__ == "__main__":
    print(build_library(force="--force" in sys.argv, verbose=True))
    print(build_host_demo(verbose=True))
