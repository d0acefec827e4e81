"""Builds ``liblingua_fp8.so`` (gfx950 only) next to this file with hipcc.

``python -m lingua_amd.build`` or ``lingua_amd.build.build()``.  The library is
built ahead of time, in-tree; nothing compiles at import or at first call.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_HERE, "liblingua_fp8.so")
SOURCES = ["api.cpp", "cast_kernels.hip", "gemm_kernels.hip", "swiglu_kernels.hip", "norm_kernels.hip"]

OBJ_DIR = os.path.join(_HERE, "build")     # object files (ignored by git)

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",      # the x * (1/scale) product must not fuse with anything
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-command-line-argument",
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass of hipcc does not know the packed-fp32 feature and says so; that is harmless
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False) -> str:
    """Compiles every source (in parallel, one object each) and links the shared library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    objs = [os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o") for src in SOURCES]
    cmds = [[hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj] for src, obj in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=min(len(cmds), os.cpu_count() or 1)) as pool:
        list(pool.map(lambda c: _run(c, verbose), cmds))
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs], verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
