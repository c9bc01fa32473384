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

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
SRC_DIR = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libscorch_hip.so")

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared",
    # packed fp32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
]


def sources():
    return sorted(glob.glob(os.path.join(SRC_DIR, "*.hip")))


def _stale() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    built = os.path.getmtime(LIB_PATH)
    deps = sources() + glob.glob(os.path.join(SRC_DIR, "*.hpp")) + [
        os.path.join(os.path.dirname(PKG_DIR), "include", "scorch_hip.h")]
    return any(os.path.getmtime(d) > built for d in deps)


def build_library(force: bool = False, verbose: bool = False) -> str:
    """Build libscorch_hip.so if it is missing or older than its sources
    (always when ``force``).  Returns the library path."""
    if not force and not _stale():
        return LIB_PATH
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("hipcc not found: cannot build libscorch_hip.so")
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc] + HIPCC_FLAGS + sources() + ["-o", tmp]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature name and says so: harmless
    noise = [l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + "\n".join(noise))
    if verbose and noise:
        print("\n".join(noise))
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    path = build_library(force="--force" in sys.argv, verbose=True)
    print(path)
