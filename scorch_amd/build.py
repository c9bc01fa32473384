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
# memory-system probes for bench.py --probe; not part of the product library
PROBES_SRC = os.path.join(SRC_DIR, "probes", "membench.hip")
PROBES_PATH = os.path.join(PKG_DIR, "libscorch_probes.so")

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared",
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


def _stale() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    built = os.path.getmtime(LIB_PATH)
    deps = sources() + glob.glob(os.path.join(SRC_DIR, "*.hpp")) + [
        os.path.join(os.path.dirname(PKG_DIR), "include", "scorch_hip.h")]
    return any(os.path.getmtime(d) > built for d in deps)


def _hipcc(srcs, out, verbose):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError(f"hipcc not found: cannot build {os.path.basename(out)}")
    tmp = out + ".tmp"
    cmd = [hipcc] + HIPCC_FLAGS + list(srcs) + ["-o", tmp]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # the host pass does not know the packed-fp32 feature name and says so: harmless
    noise = [l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l and l.strip()]
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + "\n".join(noise))
    if verbose and noise:
        print("\n".join(noise))
    os.replace(tmp, out)
    return out


def build_library(force: bool = False, verbose: bool = False) -> str:
    """Build libscorch_hip.so if it is missing or older than its sources
    (always when ``force``).  Returns the library path."""
    if not force and not _stale():
        return LIB_PATH
    return _hipcc(sources(), LIB_PATH, verbose)


def build_probes(force: bool = False, verbose: bool = False) -> str:
    """Build libscorch_probes.so (bench.py --probe) if missing, stale or forced."""
    if not force and os.path.exists(PROBES_PATH) \
            and os.path.getmtime(PROBES_PATH) >= os.path.getmtime(PROBES_SRC):
        return PROBES_PATH
    return _hipcc([PROBES_SRC], PROBES_PATH, verbose)


if __name__ == "__main__":
    print(build_library(force="--force" in sys.argv, verbose=True))
    print(build_probes(force="--force" in sys.argv, verbose=True))
