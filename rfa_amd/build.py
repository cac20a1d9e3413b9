"""Builds librfa_hip.so (the C-ABI kernel library) for gfx950 with hipcc.

Usage:  python -m rfa_amd.build [--verbose] [--resource-usage]
The library is written next to this file; it is what rfa_amd._lib loads.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "librfa_hip.so")
SOURCES = ["rfa_abi.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=fast",
    # keep the compiler from forming packed fp32 VALU ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA accumulators in VGPRs: the state tiles are re-read as operands every chunk,
    # AGPR residency would cost a v_accvgpr move per element per use
    "-mllvm", "-amdgpu-mfma-vgpr-form=1",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


def build(verbose: bool = False, extra_flags=()) -> str:
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags,
           *[os.path.join(CSRC, s) for s in SOURCES], "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


if __name__ == "__main__":
    extra = ["-Rpass-analysis=kernel-resource-usage"] if "--resource-usage" in sys.argv else []
    print(build(verbose=True if extra else ("--verbose" in sys.argv or "-v" in sys.argv), extra_flags=extra))
