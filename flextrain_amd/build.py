"""Compiles libftadam.so (the HIP kernels and their C ABI) for gfx950 with hipcc.

The library is built in-tree next to this file so that it travels with the source tree; nothing
is JIT-compiled at import time. ``python -m flextrain_amd.build`` rebuilds it.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
CSRC = os.path.join(_PKG, "csrc")
INCLUDE = os.path.join(_ROOT, "include")
LIB_PATH = os.path.join(_PKG, "libftadam.so")
SOURCES = ("ft_adam.hip", "ft_offload.hip", "ft_synth.hip")

# -ffp-contract=off: the kernels spell out every fused multiply-add; the compiler must not form
#   others, or results would differ from the reference's operation sequence.
# -packed-fp32-ops is switched off so that no v_pk_*_f32 instruction is generated.
HIPCC_FLAGS = (
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-command-line-argument",
)


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libftadam.so cannot be built")
    return exe


def build_library(verbose: bool = False, extra_flags=()) -> str:
    """Compile every HIP source and link libftadam.so. Always recompiles."""
    objs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
        cmd = [hipcc(), *HIPCC_FLAGS, *extra_flags, "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{res.stderr}")
        if verbose:
            # the host pass does not know the packed-fp32 feature and says so; that is harmless
            noise = "is not a recognized feature"
            err = "\n".join(line for line in res.stderr.splitlines() if noise not in line)
            if err.strip():
                print(err, file=sys.stderr)
        objs.append(obj)
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    return LIB_PATH


CEILING_PATH = os.path.join(_PKG, "ft_ceiling")


def build_ceiling() -> str:
    """Compile ft_ceiling: a program that times the library's kernels (the same device code, from
    the same header, with the same flags) beside bare kernels of the same memory traffic. Used by
    ``bench.py --workload ceilings`` and by the relative speed floors of the GPU tests."""
    flags = [f for f in HIPCC_FLAGS if f != "-fPIC"]
    cmd = [hipcc(), *flags, "-I", INCLUDE, "-I", CSRC, os.path.join(CSRC, "ft_ceiling.hip"), "-o", CEILING_PATH]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on ft_ceiling.hip:\n{res.stderr}")
    return CEILING_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
    print(build_ceiling())
