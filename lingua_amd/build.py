"""Builds ``liblingua_fp8.so`` (gfx950 only) next to this file with hipcc.

``python -m lingua_amd.build`` or ``lingua_amd.build.build()``.  The library is
built ahead of time, in-tree; nothing compiles at import or at first call.
"""
import os
import subprocess
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "liblingua_fp8.so")
SOURCES = ["api.cpp", "cast_kernels.hip", "gemm_kernels.hip", "swiglu_kernels.hip", "norm_kernels.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",      # the x * (1/scale) product must not fuse with anything
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def build(verbose: bool = False) -> str:
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, "-o", LIB_PATH, *[os.path.join(CSRC, s) for s in SOURCES]]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass of hipcc does not know the packed-fp32 feature and says so; that is harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
