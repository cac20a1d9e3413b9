"""Builds librfa_hip.so (the C-ABI kernel library) for gfx950 with hipcc, and
_rfa_hip_ext.so, the PyTorch C++ binding of that library (host code only, g++).

Usage:  python -m rfa_amd.build [--verbose] [--resource-usage] [--no-ext] [--only K,d -o PATH]
(--only builds a development library with the scan kernels of one (feature width, head dim) only,
in a fraction of the time, into PATH; the package never loads it by itself.)
Both are written next to this file; rfa_amd._lib loads the first with ctypes, rfa_amd.rfa_hip
imports the second when it is there.
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


def build(verbose: bool = False, extra_flags=(), out_path: str = LIB_PATH) -> str:
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags,
           *[os.path.join(CSRC, s) for s in SOURCES], "-o", out_path]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return out_path


EXT_NAME = "_rfa_hip_ext"
EXT_PATH = os.path.join(HERE, EXT_NAME + ".so")


def build_ext(verbose: bool = False) -> str:
    """The torch binding: one host C++ file compiled against torch's headers and linked to
    librfa_hip.so (found next to it at run time through $ORIGIN).  No kernels, nothing for hipcc."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension as ce
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-DTORCH_EXTENSION_NAME={EXT_NAME}",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
           "-Wno-deprecated-declarations",
           *[f"-I{p}" for p in ce.include_paths()], f"-I{sysconfig.get_paths()['include']}", f"-I{rocm}/include",
           os.path.join(CSRC, "rfa_torch_ext.cpp"), "-o", EXT_PATH,
           f"-L{torch_lib}", "-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-ltorch_python",
           f"-L{HERE}", "-l:librfa_hip.so", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building the torch binding failed:\n" + proc.stdout)
    if verbose and proc.stdout.strip():
        print(proc.stdout)
    return EXT_PATH


if __name__ == "__main__":
    extra = ["-Rpass-analysis=kernel-resource-usage"] if "--resource-usage" in sys.argv else []
    verbose = True if extra else ("--verbose" in sys.argv or "-v" in sys.argv)
    if "--only" in sys.argv:
        kd = sys.argv[sys.argv.index("--only") + 1].split(",")
        if "-o" not in sys.argv:
            sys.exit("--only needs -o PATH: a one-shape library must not replace the package's own")
        print(build(verbose=verbose, extra_flags=[*extra, f"-DRFA_ONLY_K={int(kd[0])}", f"-DRFA_ONLY_D={int(kd[1])}"],
                    out_path=sys.argv[sys.argv.index("-o") + 1]))
        sys.exit(0)
    print(build(verbose=verbose, extra_flags=extra))
    if "--no-ext" not in sys.argv and not extra:
        print(build_ext(verbose=verbose))
