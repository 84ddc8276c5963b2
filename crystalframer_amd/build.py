"""Ahead-of-time build of the HIP library for gfx950 (MI355X).

The reference compiles its kernels at run time with NVRTC after text substitution
(models/cuda_funcs/kernel_manager.py:116-167); here every supported constant set is a template
instantiation compiled once by hipcc into ``libcrystalframer_hip.so`` next to this file.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_NAME = "libcrystalframer_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)

HIPCC_FLAGS = [
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-shared", "-fPIC",
    # packed FP32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")


def build_library(verbose: bool = True) -> str:
    """Compile csrc/crystalframer_hip.hip -> libcrystalframer_hip.so (always recompiles)."""
    src = os.path.join(CSRC, "crystalframer_hip.hip")
    tmp = LIB_PATH + ".tmp"
    # CFH_EXTRA_HIPCC_FLAGS: extra flags for diagnostics builds (e.g. -DCFH_PHASE_TIMING)
    extra = os.environ.get("CFH_EXTRA_HIPCC_FLAGS", "").split()
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra, "-o", tmp, src]
    if verbose:
        print("[crystalframer_amd] " + " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout + res.stderr)
        raise RuntimeError("hipcc failed building " + LIB_NAME)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
