"""Builds ``liblingua_fp8.so`` (gfx950 only) next to this file with hipcc.

``python -m lingua_amd.build`` or ``lingua_amd.build.build()``.  The library is
built ahead of time, in-tree; nothing compiles at import or at first call.
"""
import os
import re
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
# LINGUA_FP8_LIB: where to put the library instead (a tuning variant beside the shipped one; `lingua_amd._lib` reads the
# same variable); LINGUA_FP8_HIPCC_EXTRA: more hipcc flags for such a variant, e.g. "-DL8_STRADDLE=3 -DL8_READ_GROUPS=10".
LIB_PATH = os.environ.get("LINGUA_FP8_LIB") or os.path.join(_HERE, "liblingua_fp8.so")
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
    """Runs one hipcc command; returns the register / scratch figures of the kernels it compiled
    ({mangled name: {"VGPRs": n, "AGPRs": n, "ScratchSize": bytes per lane, "VGPRs Spill": n, "SGPRs Spill": n}})."""
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    usage, cur, rest = {}, None, []
    for line in res.stderr.splitlines():
        if "packed-fp32-ops" in line:
            continue  # the host pass of hipcc does not know the packed-fp32 feature and says so; that is harmless
        if "[-Rpass-analysis=kernel-resource-usage]" in line:
            m = re.search(r"Function Name: (\S+)", line)
            if m:
                cur = usage.setdefault(m.group(1), {})
            m = re.search(r"remark:\s+(VGPRs Spill|SGPRs Spill|ScratchSize|VGPRs|AGPRs)(?: \[[^\]]*\])?: (\d+)", line)
            if m and cur is not None:
                cur[m.group(1)] = int(m.group(2))
            continue
        rest.append(line)
    err = "\n".join(rest)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    return usage


def _check_usage(usage) -> None:
    """The persistent GEMM kernel runs at the edge of the register file: a source change that makes the allocator
    spill (or leaves loop state in private memory, which turns every panel load into a loop over lanes) costs a
    third of its speed and no test would notice.  Such a build fails here instead -- and so does a build whose
    compiler remarks could not be read (no entry for the kernel, or an entry without the scratch figure): a check
    that finds nothing to check must not pass."""
    stream = {name: u for name, u in usage.items() if "gemm_nt_stream_kernel" in name}
    if not stream:
        raise RuntimeError("no register / scratch remarks were parsed for the persistent GEMM kernel "
                           "(-Rpass-analysis=kernel-resource-usage output missing or in a new format)")
    unread = [name for name, u in stream.items() if "ScratchSize" not in u or "VGPRs Spill" not in u]
    if unread:
        raise RuntimeError("resource remarks without scratch / spill figures for:\n  " + "\n  ".join(unread))
    bad = [f"{name}: {u}" for name, u in stream.items() if (u["ScratchSize"] or u["VGPRs Spill"])]
    if bad:
        raise RuntimeError("the persistent GEMM kernel must not use scratch memory:\n  " + "\n  ".join(bad))
    # The cast, gate and norm kernels stream memory with several loads in flight per lane; a reload from scratch memory
    # waits for every one of them (loads retire in order).  None of them needs scratch, so one that starts to is a
    # regression of the source.  (The plain GEMM kernels of the non-default tile configurations spill a few registers
    # by design and are not checked.)
    bad = [f"{name}: {u}" for name, u in usage.items()
           if "gemm_nt" not in name and (u.get("ScratchSize") or u.get("VGPRs Spill"))]
    if bad:
        raise RuntimeError("memory-streaming kernels must not use scratch memory:\n  " + "\n  ".join(bad))


def build(verbose: bool = False) -> str:
    """Compiles every source (in parallel, one object each) and links the shared library."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    extra = os.environ.get("LINGUA_FP8_HIPCC_EXTRA", "").split()
    obj_dir = OBJ_DIR if not os.environ.get("LINGUA_FP8_LIB") else os.path.join(OBJ_DIR, os.path.splitext(os.path.basename(LIB_PATH))[0])
    os.makedirs(obj_dir, exist_ok=True)
    objs = [os.path.join(obj_dir, os.path.splitext(src)[0] + ".o") for src in SOURCES]
    cmds = [[hipcc, *HIPCC_FLAGS, *extra, *(["-Rpass-analysis=kernel-resource-usage"] if src.endswith(".hip") else []),
             "-c", os.path.join(CSRC, src), "-o", obj] for src, obj in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=min(len(cmds), os.cpu_count() or 1)) as pool:
        usages = list(pool.map(lambda c: _run(c, verbose), cmds))
    usage = {k: v for u in usages for k, v in u.items()}
    with open(os.path.join(obj_dir, "resource_usage.txt"), "w") as f:
        for name in sorted(usage):
            f.write(f"{name} {usage[name]}\n")
    _check_usage(usage)
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs], verbose)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
