"""CPU oracle for the row-wise float8 linear recipe -- TEST INFRASTRUCTURE ONLY.

Only the tests, the smoke test and the benchmark's ``cpu_baseline`` leg may
import this package; the shipped ``lingua_amd`` package never does.

Two independent restatements of the reference algorithm live here:

* ``fp8_recipe_oracle.c`` (bound below through ctypes): integer-exact C.
* ``recipe_torch`` : the same recipe as a chain of PyTorch CPU ops, in the
  order the reference issues them (lingua/float8.py:43-47, 50-79, 85-131).

They are checked against each other and against independent facts in
``tests/test_oracle_*.py``.
"""
import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libl8oracle.so")
_lib = None

_i64 = ctypes.c_int64
_p = ctypes.c_void_p


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B", "libl8oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        L.l8o_e4m3fn_from_f32_bits.restype = ctypes.c_uint8
        L.l8o_e4m3fn_from_f32_bits.argtypes = [ctypes.c_uint32]
        L.l8o_e4m3fn_to_f32.restype = ctypes.c_float
        L.l8o_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        L.l8o_scale_from_amax.restype = ctypes.c_float
        L.l8o_scale_from_amax.argtypes = [ctypes.c_uint16]
        L.l8o_amax_of_amaxes.restype = ctypes.c_uint16
        L.l8o_amax_of_amaxes.argtypes = [_p, _i64]
        L.l8o_f32_to_bf16.restype = ctypes.c_uint16
        L.l8o_f32_to_bf16.argtypes = [ctypes.c_float]
        L.l8o_row_amax.argtypes = [_p, _i64, _i64, _i64, _p]
        L.l8o_col_amax.argtypes = [_p, _i64, _i64, _i64, _p]
        L.l8o_cast_rowwise.argtypes = [_p, _i64, _i64, _i64, _p, _i64, _p, _p]
        L.l8o_cast_tensorwise.argtypes = [_p, _i64, _i64, _i64, ctypes.c_uint16, ctypes.c_int, _p, _i64, _p]
        L.l8o_cast_colwise_transposed.argtypes = [_p, _i64, _i64, _i64, _p, _p, _i64, _p]
        L.l8o_gemm_nt.argtypes = [_p, _p, _i64, _i64, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _p, _i64]
        L.l8o_gemm_nt_f64.argtypes = [_p, _p, _i64, _i64, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _p, _i64]
        L.l8o_col_sum.argtypes = [_p, _i64, _i64, _i64, _p]
        L.l8o_e4m3fn_from_f32_array.argtypes = [_p, _i64, _p]
        L.l8o_scale_from_amax_array.argtypes = [_p, _i64, _p]
        L.l8o_set_scale_rule.argtypes = [ctypes.c_int]
        L.l8o_set_scale_rule.restype = None
        L.l8o_get_scale_rule.restype = ctypes.c_int
        for name in ("l8o_row_amax", "l8o_col_amax", "l8o_cast_rowwise", "l8o_cast_tensorwise",
                     "l8o_cast_colwise_transposed", "l8o_gemm_nt", "l8o_gemm_nt_f64", "l8o_col_sum",
                     "l8o_e4m3fn_from_f32_array", "l8o_scale_from_amax_array"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


class scale_rule:
    """``with oracle.scale_rule("times_inverse"):`` -- both restatements evaluate ``clamp(amax) / 448`` the way
    ATen's GPU kernel does (product with fp32(1/448)) instead of the correctly rounded quotient of ATen's CPU kernel
    ("divide", the default)."""
    RULES = {"divide": 0, "times_inverse": 1}

    def __init__(self, rule: str):
        self.rule = self.RULES[rule]

    def __enter__(self):
        from . import recipe_torch
        self.before = lib().l8o_get_scale_rule()
        lib().l8o_set_scale_rule(self.rule)
        recipe_torch.SCALE_TIMES_INVERSE = bool(self.rule)
        return self

    def __exit__(self, *exc):
        from . import recipe_torch
        lib().l8o_set_scale_rule(self.before)
        recipe_torch.SCALE_TIMES_INVERSE = bool(self.before)
        return False


# ----------------------------------------------------------------------------
# tensor helpers: everything below takes / returns CPU torch tensors
# ----------------------------------------------------------------------------

def _bf16_2d(t: torch.Tensor) -> torch.Tensor:
    assert t.dtype == torch.bfloat16 and t.dim() == 2 and t.device.type == "cpu"
    return t.contiguous()


def _u8(t: torch.Tensor) -> torch.Tensor:
    if t.dtype == torch.float8_e4m3fn:
        t = t.view(torch.uint8)
    assert t.dtype == torch.uint8 and t.device.type == "cpu"
    return t.contiguous()


def e4m3fn_from_f32(x: torch.Tensor) -> torch.Tensor:
    """Elementwise fp32 -> e4m3fn bytes (uint8), through the integer routine."""
    w = x.detach().to(torch.float32).contiguous().view(torch.int32)
    out = torch.empty(w.shape, dtype=torch.uint8)
    lib().l8o_e4m3fn_from_f32_array(w.data_ptr(), w.numel(), out.data_ptr())
    return out


def e4m3fn_decode_table() -> torch.Tensor:
    L = lib()
    return torch.tensor([L.l8o_e4m3fn_to_f32(i) for i in range(256)], dtype=torch.float32)


def scale_from_amax(amax: torch.Tensor) -> torch.Tensor:
    """bf16 amax tensor -> fp32 scale tensor (same shape)."""
    a = amax.detach().to(torch.bfloat16).contiguous()
    out = torch.empty(a.shape, dtype=torch.float32)
    lib().l8o_scale_from_amax_array(a.data_ptr(), a.numel(), out.data_ptr())
    return out


def row_amax(x: torch.Tensor) -> torch.Tensor:
    x = _bf16_2d(x)
    R, C = x.shape
    out = torch.empty(R, dtype=torch.bfloat16)
    lib().l8o_row_amax(x.data_ptr(), R, C, C, out.data_ptr())
    return out


def col_amax(x: torch.Tensor) -> torch.Tensor:
    x = _bf16_2d(x)
    R, C = x.shape
    out = torch.empty(C, dtype=torch.bfloat16)
    lib().l8o_col_amax(x.data_ptr(), R, C, C, out.data_ptr())
    return out


def amax_of_amaxes(amax: torch.Tensor) -> torch.Tensor:
    a = amax.detach().to(torch.bfloat16).contiguous().reshape(-1)
    bits = lib().l8o_amax_of_amaxes(a.data_ptr(), a.numel())
    return torch.tensor([bits], dtype=torch.int32).to(torch.int16).view(torch.bfloat16).reshape(())


def cast_rowwise(x: torch.Tensor):
    """-> (q uint8 [R,C], scale fp32 [R], amax bf16 [R])"""
    x = _bf16_2d(x)
    R, C = x.shape
    q = torch.empty(R, C, dtype=torch.uint8)
    s = torch.empty(R, dtype=torch.float32)
    a = torch.empty(R, dtype=torch.bfloat16)
    lib().l8o_cast_rowwise(x.data_ptr(), R, C, C, q.data_ptr(), C, s.data_ptr(), a.data_ptr())
    return q, s, a


def cast_tensorwise(x: torch.Tensor, amax: torch.Tensor = None, transpose: bool = False):
    """-> (q uint8 [R,C] or [C,R], scale fp32 [1]).  amax: bf16 scalar (default: of x)."""
    x = _bf16_2d(x)
    R, C = x.shape
    if amax is None:
        amax = amax_of_amaxes(row_amax(x))
    bits = int(amax.detach().to(torch.bfloat16).reshape(1).view(torch.int16).item()) & 0xFFFF
    q = torch.empty((C, R) if transpose else (R, C), dtype=torch.uint8)
    s = torch.empty(1, dtype=torch.float32)
    lib().l8o_cast_tensorwise(x.data_ptr(), R, C, C, bits, int(transpose), q.data_ptr(), q.shape[1], s.data_ptr())
    return q, s


def cast_colwise_transposed(x: torch.Tensor, amax: torch.Tensor = None):
    """scale(x.t().contiguous(), its row amax) -> (q uint8 [C,R], scale fp32 [C])"""
    x = _bf16_2d(x)
    R, C = x.shape
    q = torch.empty(C, R, dtype=torch.uint8)
    s = torch.empty(C, dtype=torch.float32)
    ap = None
    if amax is not None:
        amax = amax.detach().to(torch.bfloat16).contiguous().reshape(-1)
        assert amax.numel() == C
        ap = amax.data_ptr()
    lib().l8o_cast_colwise_transposed(x.data_ptr(), R, C, C, ap, q.data_ptr(), R, s.data_ptr())
    return q, s


def gemm_nt(qa, qb, sa, sb, bias=None, f64=False):
    """bf16( (qa*sa) @ (qb*sb)^T + bias ), fp32 accumulation.  sa: [M] or [1]; sb: [N] or [1]."""
    qa, qb = _u8(qa), _u8(qb)
    M, K = qa.shape
    N, K2 = qb.shape
    assert K == K2
    sa = sa.detach().to(torch.float32).contiguous().reshape(-1)
    sb = sb.detach().to(torch.float32).contiguous().reshape(-1)
    assert sa.numel() in (1, M) and sb.numel() in (1, N)
    bp = None
    if bias is not None:
        bias = bias.detach().to(torch.bfloat16).contiguous()
        assert bias.numel() == N
        bp = bias.data_ptr()
    if f64:
        out = torch.empty(M, N, dtype=torch.float64)
        fn = lib().l8o_gemm_nt_f64
    else:
        out = torch.empty(M, N, dtype=torch.bfloat16)
        fn = lib().l8o_gemm_nt
    fn(qa.data_ptr(), qb.data_ptr(), M, N, K, K, K, sa.data_ptr(), sa.numel(), sb.data_ptr(), sb.numel(),
       bp, out.data_ptr(), N)
    return out


def col_sum(g: torch.Tensor) -> torch.Tensor:
    g = _bf16_2d(g)
    R, C = g.shape
    out = torch.empty(C, dtype=torch.bfloat16)
    lib().l8o_col_sum(g.data_ptr(), R, C, C, out.data_ptr())
    return out


# ----------------------------------------------------------------------------
# the three products of one linear, as the reference recipe defines them
# ----------------------------------------------------------------------------

def linear_forward(a, w, bias=None):
    """lingua/float8.py:85-96 : both operands row-wise."""
    qa, sa, _ = cast_rowwise(a)
    qw, sw, _ = cast_rowwise(w)
    return gemm_nt(qa, qw, sa, sw, bias)


def linear_dgrad(grad_out, w):
    """lingua/float8.py:110-119 : grad_out row-wise, weight tensor-wise (from its row amaxes)."""
    qg, sg, _ = cast_rowwise(grad_out)
    qwt, sw = cast_tensorwise(w, amax_of_amaxes(row_amax(w)), transpose=True)
    return gemm_nt(qg, qwt, sg, sw)


def linear_wgrad_fp8(grad_out, a):
    """fp8 wgrad: both operands quantised along the token dimension (not in the
    reference, whose wgrad is a bf16 matmul, lingua/float8.py:123)."""
    qgt, sgt = cast_colwise_transposed(grad_out)
    qat, sat = cast_colwise_transposed(a)
    return gemm_nt(qgt, qat, sgt, sat)
