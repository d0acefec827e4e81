"""ctypes binding of ``liblingua_fp8.so`` (declared in ``include/lingua_fp8.h``).

There is exactly one implementation: if the shared library is missing, or the
GPU is not a gfx950 part, every op raises.  Nothing here falls back to PyTorch
ops or to the CPU.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
# LINGUA_FP8_LIB names another build of the library (a tuning variant made with `python -m lingua_amd.build` under the
# same variable); unset, the library next to this file is the one that is loaded.
LIB_PATH = os.environ.get("LINGUA_FP8_LIB") or os.path.join(_HERE, "liblingua_fp8.so")

_i64 = ctypes.c_int64
_int = ctypes.c_int
_p = ctypes.c_void_p

# name -> argtypes; every function returns int except where noted
SIGNATURES = {
    "l8_version": [],
    "l8_last_error": [],
    "l8_device_check": [_int],
    "l8_set_scale_rule": [_int],
    "l8_get_scale_rule": [],
    "l8_cast_rowwise": [_p, _i64, _i64, _i64, _p, _i64, _p, _p, _p, _p, _i64, _p],
    "l8_cast_rowwise_workspace": [_i64, _i64],
    "l8_cast_rowwise_noalloc": [_p, _i64, _i64, _i64, _p, _i64, _p, _p, _p, _p],
    "l8_cast_rowwise_given_amax": [_p, _i64, _i64, _i64, _p, _int, _p, _i64, _p, _p],
    "l8_col_amax": [_p, _i64, _i64, _i64, _p, _p],
    "l8_amax_reduce": [_p, _i64, _p, _p],
    "l8_cast_tensorwise": [_p, _i64, _i64, _i64, _p, _int, _int, _p, _i64, _p, _p],
    "l8_cast_colwise_transposed": [_p, _i64, _i64, _i64, _p, _p, _i64, _p, _p],
    "l8_gemm_nt": [_p, _p, _i64, _i64, _i64, _i64, _i64, _p, _int, _p, _int, _p, _p, _i64, _int, _p],
    "l8_gemm_nt_ws": [_p, _p, _i64, _i64, _i64, _i64, _i64, _p, _int, _p, _int, _p, _p, _i64, _int, _p, _i64, _p],
    "l8_gemm_workspace": [],
    "l8_gemm_workspace_gave_up_offset": [],
    "l8_gemm_set_wait_limit": [_int],
    "l8_gemm_shares_k": [_i64, _i64, _i64, _int],
    "l8_swiglu_cast_rowwise": [_p, _p, _i64, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _p, _p, _p, _i64, _p],
    "l8_swiglu_workspace": [_i64, _i64],
    "l8_swiglu_bwd_cast_rowwise": [_p, _p, _p, _i64, _i64, _i64, _i64, _i64, _p, _p, _i64, _p, _p, _i64, _p, _p, _p, _p,
                                   _p, _i64, _p],
    "l8_rmsnorm_cast_rowwise": [_p, _p, _int, _i64, _i64, _i64, ctypes.c_float, _p, _i64, _p, _i64, _p, _p, _p, _p, _i64, _p],
    "l8_rmsnorm_workspace": [_i64, _i64],
    "l8_rmsnorm_bwd": [_p, _p, _p, _int, _p, _i64, _i64, _i64, _i64, _p, _i64, _p, _p, _i64, _p],
    "l8_rmsnorm_bwd_workspace": [_i64, _i64],
    "l8_gemm_algo_count": [],
    "l8_gemm_algo_name": [_int],
    "l8_gemm_pick": [_i64, _i64, _i64],
}
_RETURNS_STR = {"l8_last_error", "l8_gemm_algo_name"}
_RETURNS_I64 = {"l8_cast_rowwise_workspace", "l8_gemm_workspace", "l8_gemm_workspace_gave_up_offset", "l8_swiglu_workspace", "l8_rmsnorm_workspace", "l8_rmsnorm_bwd_workspace"}

_lib = None
_lock = threading.Lock()
_checked_devices = set()


def load():
    """Load the library (once). Raises RuntimeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with `python -m lingua_amd.build` "
                    "(there is no fallback implementation)"
                )
            lib = ctypes.CDLL(LIB_PATH)
            for name, argtypes in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.argtypes = argtypes
                fn.restype = ctypes.c_char_p if name in _RETURNS_STR else (_i64 if name in _RETURNS_I64 else _int)
            _lib = lib
    return _lib


def last_error() -> str:
    msg = load().l8_last_error()
    return msg.decode() if msg else ""


def check(code: int, what: str) -> None:
    if code != 0:
        raise RuntimeError(f"{what} failed ({code}): {last_error()}")


def require_device(index: int) -> None:
    """Raise unless HIP device ``index`` is gfx950 (checked once per device)."""
    if index in _checked_devices:
        return
    check(load().l8_device_check(index), "l8_device_check")
    _checked_devices.add(index)
