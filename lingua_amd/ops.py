"""Tensor-level wrappers around the C ABI: shape checks, output allocation
(by PyTorch's caching allocator, on the current stream) and the call itself.

All inputs are CUDA (HIP) tensors on a gfx950 device.  Outputs are returned as
``torch.float8_e4m3fn`` / ``torch.float32`` / ``torch.bfloat16`` tensors.
"""
from typing import Optional, Tuple

import torch

from . import _lib

SCALE_SCALAR = 0
SCALE_ROW = 1

# Optional per-kernel timing: when `kernel_timer` is a list, every launch below
# appends (kernel name, start event, end event, algorithmic work) where the
# events are recorded on the stream the kernel runs on.  Work is flop for the
# GEMM and compulsory bytes for the casts.  None (the default) records nothing.
# `kernel_timer_names` (a set of kernel names, or None for all) limits the recording: every pair of events costs
# the stream a little, which a caller timing a whole step may not want to pay for every launch.
kernel_timer = None
kernel_timer_names = None


class _timed:
    """Brackets one launch: makes the tensor's device current for its duration (the library launches on the
    current device; the caller's current device is restored afterwards) and, when `kernel_timer` is a list,
    records the two events."""
    __slots__ = ("name", "work", "dev", "ev", "prev")

    def __init__(self, name, work, dev):
        self.name, self.work, self.dev, self.ev, self.prev = name, work, dev, None, None

    def __enter__(self):
        cur = torch.cuda.current_device()
        if self.dev.index is not None and self.dev.index != cur:
            self.prev = cur
            torch.cuda.set_device(self.dev)
        if kernel_timer is not None and (kernel_timer_names is None or self.name in kernel_timer_names):
            self.ev = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            self.ev[0].record(torch.cuda.current_stream(self.dev))

    def __exit__(self, *exc):
        if self.ev is not None:
            self.ev[1].record(torch.cuda.current_stream(self.dev))
            kernel_timer.append((self.name, self.ev[0], self.ev[1], self.work))
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False


def _prep(t: torch.Tensor, what: str):
    """Checks that `t` lives on a gfx950 GPU and returns the raw handle of the calling thread's current stream
    on that GPU.  The process's current device is left alone."""
    if not t.is_cuda:
        raise RuntimeError(f"{what}: expected a GPU tensor, got device {t.device} (there is no CPU path)")
    _lib.require_device(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


def _wrote_into(t: torch.Tensor) -> None:
    """A kernel has written into caller-supplied memory through its raw pointer: advance the tensor's version
    counter, as an in-place PyTorch op would, so that autograd's saved-tensor check and the cast memo of
    lingua_amd.float8 see the write."""
    if not t.is_inference():
        torch.autograd.graph.increment_version(t)


def _rows_2d(t: torch.Tensor, dtype, what: str) -> torch.Tensor:
    if t.dtype != dtype or t.dim() != 2:
        raise RuntimeError(f"{what}: expected a 2-D {dtype} tensor, got {t.dtype} {tuple(t.shape)}")
    if t.numel() and (t.stride(1) != 1 or t.stride(0) < t.shape[1]):
        t = t.contiguous()
    return t


def _ld(t: torch.Tensor) -> int:
    return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], 1)


def cast_rowwise(x: torch.Tensor, col_amax: Optional[torch.Tensor] = None, want_q: bool = True,
                 out_q: Optional[torch.Tensor] = None, out_scale: Optional[torch.Tensor] = None):
    """Row-wise amax -> scale -> e4m3fn.  Returns (q [R,C] fp8 | None, scale [R,1] fp32, amax [R,1] bf16).

    ``col_amax`` (fp32 [C]) receives the column amaxes of x (overwritten).
    ``out_q`` (fp8 [R,C], unit column stride, row stride a multiple of 8) and ``out_scale`` (fp32 [R,1], any
    strides) receive the results in place of fresh tensors: a column slice of a wider matrix is the use."""
    x = _rows_2d(x, torch.bfloat16, "cast_rowwise")
    st = _prep(x, "cast_rowwise")
    R, C = x.shape
    q = None
    if want_q:
        q = out_q if out_q is not None else torch.empty((R, C), dtype=torch.float8_e4m3fn, device=x.device)
        if q.dtype != torch.float8_e4m3fn or tuple(q.shape) != (R, C) or q.device != x.device or (q.numel() and q.stride(1) != 1):
            raise RuntimeError("cast_rowwise: out_q must be an e4m3fn [R,C] tensor on x's device with unit column stride")
    if out_scale is not None and (out_scale.dtype != torch.float32 or tuple(out_scale.shape) != (R, 1) or out_scale.device != x.device):
        raise RuntimeError("cast_rowwise: out_scale must be fp32 [R,1] on x's device")
    scale_direct = out_scale is not None and (R <= 1 or out_scale.stride(0) == 1)  # the kernel writes a dense vector
    scale = out_scale if scale_direct else torch.empty((R, 1), dtype=torch.float32, device=x.device)
    amax = torch.empty((R, 1), dtype=torch.bfloat16, device=x.device)
    if col_amax is not None and (col_amax.dtype != torch.float32 or col_amax.numel() != C or not col_amax.is_contiguous()):
        raise RuntimeError("cast_rowwise: col_amax must be a contiguous fp32 tensor with C elements")
    ws, ws_bytes = None, 0
    if col_amax is not None:
        ws_bytes = _lib.load().l8_cast_rowwise_workspace(R, C)
        if ws_bytes:
            ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device)
    with _timed("cast_rowwise", R * C * (3 if want_q else 2) + 4 * R + (4 * C if col_amax is not None else 0), x.device):
        code = _lib.load().l8_cast_rowwise(
            x.data_ptr(), R, C, _ld(x), q.data_ptr() if want_q else None, _ld(q) if want_q else C, scale.data_ptr(),
            amax.data_ptr(), col_amax.data_ptr() if col_amax is not None else None,
            ws.data_ptr() if ws is not None else None, ws_bytes, st)
    _lib.check(code, "l8_cast_rowwise")
    if out_q is not None and want_q:
        _wrote_into(out_q)
    if scale_direct:
        _wrote_into(out_scale)
    elif out_scale is not None:
        scale = out_scale.copy_(scale)
    return q, scale, amax


AMAX_BF16, AMAX_F32 = 0, 1


def _amax_arg(amax: torch.Tensor, n: int, device, what: str):
    """An amax handed in by the caller, as the kernels take it: bf16 and fp32 as they are (the reference converts
    with ``.float()``, lingua/float8.py:44, which is exact for both), any other floating dtype through fp32."""
    if not amax.is_floating_point() or amax.numel() != n or amax.device != device:
        raise RuntimeError(f"{what}: amax must be a floating-point tensor with {n} element(s) on the input's device")
    if amax.dtype not in (torch.bfloat16, torch.float32):
        amax = amax.float()
    return amax.contiguous(), (AMAX_F32 if amax.dtype == torch.float32 else AMAX_BF16)


def cast_rowwise_given_amax(x: torch.Tensor, amax: torch.Tensor):
    """scale(x, amax) of lingua/float8.py:43-47 with a row amax [R,1] (bf16 or fp32) the caller supplies and that is
    used as given.  Returns (q [R,C] fp8, scale [R,1] fp32)."""
    x = _rows_2d(x, torch.bfloat16, "cast_rowwise_given_amax")
    st = _prep(x, "cast_rowwise_given_amax")
    R, C = x.shape
    amax, amax_dtype = _amax_arg(amax, R, x.device, "cast_rowwise_given_amax")
    q = torch.empty((R, C), dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((R, 1), dtype=torch.float32, device=x.device)
    with _timed("cast_rowwise_given_amax", R * C * 3 + 6 * R, x.device):
        code = _lib.load().l8_cast_rowwise_given_amax(x.data_ptr(), R, C, _ld(x), amax.data_ptr(), amax_dtype, q.data_ptr(), C,
                                                      scale.data_ptr(), st)
    _lib.check(code, "l8_cast_rowwise_given_amax")
    return q, scale


def col_amax(x: torch.Tensor) -> torch.Tensor:
    """fp32 [C] column amaxes of bf16 x [R,C]."""
    x = _rows_2d(x, torch.bfloat16, "col_amax")
    st = _prep(x, "col_amax")
    R, C = x.shape
    out = torch.empty(C, dtype=torch.float32, device=x.device)
    with _timed("col_amax", R * C * 2 + 4 * C, x.device):
        code = _lib.load().l8_col_amax(x.data_ptr(), R, C, _ld(x), out.data_ptr(), st)
    _lib.check(code, "l8_col_amax")
    return out


def amax_reduce(amax: torch.Tensor) -> torch.Tensor:
    """bf16 [n] (any shape) -> bf16 [1,1] max, NaN propagating."""
    if amax.dtype != torch.bfloat16:
        raise RuntimeError("amax_reduce: expected bf16")
    amax = amax.contiguous()
    st = _prep(amax, "amax_reduce")
    out = torch.empty((1, 1), dtype=torch.bfloat16, device=amax.device)
    with _timed("amax_reduce", 2 * amax.numel() + 2, amax.device):
        code = _lib.load().l8_amax_reduce(amax.data_ptr(), amax.numel(), out.data_ptr(), st)
    _lib.check(code, "l8_amax_reduce")
    return out


def cast_tensorwise(x: torch.Tensor, amax: torch.Tensor, transpose: bool = False):
    """Tensor-wise scale -> e4m3fn with a device-resident amax scalar (bf16 or fp32).
    Returns (q [R,C] or [C,R] fp8, scale [1,1] fp32)."""
    x = _rows_2d(x, torch.bfloat16, "cast_tensorwise")
    st = _prep(x, "cast_tensorwise")
    amax, amax_dtype = _amax_arg(amax, 1, x.device, "cast_tensorwise")
    R, C = x.shape
    q = torch.empty((C, R) if transpose else (R, C), dtype=torch.float8_e4m3fn, device=x.device)
    scale = torch.empty((1, 1), dtype=torch.float32, device=x.device)
    with _timed("cast_tensorwise_t" if transpose else "cast_tensorwise", R * C * 3 + 4, x.device):
        code = _lib.load().l8_cast_tensorwise(x.data_ptr(), R, C, _ld(x), amax.data_ptr(), amax_dtype, int(transpose),
                                              q.data_ptr(), max(q.shape[1], 1), scale.data_ptr(), st)
    _lib.check(code, "l8_cast_tensorwise")
    return q, scale


def cast_colwise_transposed(x: torch.Tensor, col_amax_f32: torch.Tensor, pad_to: int = 16):
    """scale(x.t().contiguous(), its row amax): returns (q [C,Rp] fp8, scale [C,1] fp32).

    Rp is R rounded up to a multiple of ``pad_to``; the padding columns hold
    e4m3 zeros, so a product whose reduction runs over them is unchanged (the
    GEMM needs a reduction length that is a multiple of 16, token counts are
    arbitrary)."""
    x = _rows_2d(x, torch.bfloat16, "cast_colwise_transposed")
    st = _prep(x, "cast_colwise_transposed")
    R, C = x.shape
    if col_amax_f32.dtype != torch.float32 or col_amax_f32.numel() != C or not col_amax_f32.is_contiguous():
        raise RuntimeError("cast_colwise_transposed: col_amax must be a contiguous fp32 tensor with C elements")
    if R == 0:
        # no rows: the product over them is zero; one block of zero columns keeps the GEMM's reduction length valid
        q = torch.zeros((C, pad_to), dtype=torch.uint8, device=x.device).view(torch.float8_e4m3fn)
        return q, (torch.clamp(col_amax_f32, min=1e-12) / 448.0).reshape(C, 1)
    Rp = (R + pad_to - 1) // pad_to * pad_to
    q = torch.empty((C, Rp), dtype=torch.float8_e4m3fn, device=x.device)
    if Rp != R:
        q.view(torch.uint8)[:, R:].zero_()   # the kernel writes columns 0 .. R-1; only the padding is filled here
    scale = torch.empty((C, 1), dtype=torch.float32, device=x.device)
    with _timed("cast_colwise_t", R * C * 3 + 4 * C, x.device):
        code = _lib.load().l8_cast_colwise_transposed(x.data_ptr(), R, C, _ld(x), col_amax_f32.data_ptr(),
                                                      q.data_ptr(), max(Rp, 1), scale.data_ptr(), st)
    _lib.check(code, "l8_cast_colwise_transposed")
    return q, scale


# Tile configuration that may share the K range of the last round's tiles out (opt-in: measured neutral), and its
# workspace: one per (device, stream), zero-filled when it is made, then owned by the library.
GEMM_ALGO_SHARED_K = 15
_gemm_workspaces = {}


def _gemm_workspace(device: torch.device, stream_ptr, algo: int):
    if algo != GEMM_ALGO_SHARED_K:
        return None, 0
    key = (device.index, stream_ptr)
    ws = _gemm_workspaces.get(key)
    if ws is None:
        if torch.cuda.is_current_stream_capturing():
            return None, 0  # no allocation (and no fill) inside a capture; the library takes its plain path
        ws = torch.zeros(_lib.load().l8_gemm_workspace(), dtype=torch.uint8, device=device)
        _gemm_workspaces[key] = ws
    return ws.data_ptr(), ws.numel()


def shared_k_tiles_given_up(device=None) -> int:
    """Number of tiles that tile configuration 15 stored as NaNs since its workspaces on `device` were made,
    because their owners' bounded wait for a helper's partial sums ran out (the call itself cannot report it).
    Synchronises the device.  0 is the only healthy answer."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    off = _lib.load().l8_gemm_workspace_gave_up_offset()
    total = 0
    torch.cuda.synchronize(dev)
    for (index, _), ws in list(_gemm_workspaces.items()):
        if index == dev.index:
            total += int(ws[off:off + 4].view(torch.int32).item())
    return total


def release_gemm_workspaces() -> None:
    """Frees the workspaces of tile configuration 15 (64 MiB per (device, stream) that used it; otherwise they
    live as long as the process).  The next call that needs one makes it afresh."""
    _gemm_workspaces.clear()


def gemm_nt(qa: torch.Tensor, qb: torch.Tensor, sa: torch.Tensor, sb: torch.Tensor,
            bias: Optional[torch.Tensor] = None, algo: int = 0, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """bf16( (qa @ qb^T) * sa * sb^T + bias ).  qa [M,K], qb [N,K] fp8; sa [M,1]|[1,1], sb [N,1]|[1,1] fp32."""
    qa = _rows_2d(qa, torch.float8_e4m3fn, "gemm_nt(A)")
    qb = _rows_2d(qb, torch.float8_e4m3fn, "gemm_nt(B)")
    st = _prep(qa, "gemm_nt")
    M, K = qa.shape
    N, K2 = qb.shape
    if K != K2:
        raise RuntimeError(f"gemm_nt: reduction dims differ ({K} vs {K2})")
    if sa.dtype != torch.float32 or sb.dtype != torch.float32 or sa.numel() not in (1, M) or sb.numel() not in (1, N):
        raise RuntimeError("gemm_nt: scales must be fp32 with 1 or M (resp. N) elements")
    sa, sb = sa.contiguous(), sb.contiguous()
    sa_mode = SCALE_ROW if sa.numel() == M else SCALE_SCALAR
    sb_mode = SCALE_ROW if sb.numel() == N else SCALE_SCALAR
    if bias is not None:
        if bias.dtype != torch.bfloat16 or bias.numel() != N:
            raise RuntimeError("gemm_nt: bias must be bf16 with N elements")
        bias = bias.contiguous()
    user_out = out is not None
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=qa.device)
    elif out.dtype != torch.bfloat16 or out.shape != (M, N) or out.stride(1) != 1:
        raise RuntimeError("gemm_nt: out must be bf16 [M,N] with unit column stride")
    ws_ptr, ws_bytes = _gemm_workspace(qa.device, st, algo)
    with _timed("gemm_nt", 2 * M * N * K, qa.device):
        code = _lib.load().l8_gemm_nt_ws(qa.data_ptr(), qb.data_ptr(), M, N, K, _ld(qa), _ld(qb), sa.data_ptr(), sa_mode,
                                         sb.data_ptr(), sb_mode, bias.data_ptr() if bias is not None else None,
                                         out.data_ptr(), _ld(out) if M > 1 else max(N, 1), algo, ws_ptr, ws_bytes, st)
    _lib.check(code, "l8_gemm_nt_ws")
    if user_out:
        _wrote_into(out)
    return out


def gemm_pick(M: int, N: int, K: int) -> Tuple[int, str]:
    """(number, name) of the tile configuration that ``algo=0`` resolves to for an M x N x K problem on the current
    device (aligned operands assumed)."""
    lib = _lib.load()
    algo = lib.l8_gemm_pick(M, N, K)
    if algo <= 0:
        _lib.check(algo, "l8_gemm_pick")
    return algo, lib.l8_gemm_algo_name(algo).decode()


SCALE_RULES = {"divide": 0, "times_inverse": 1}


def set_scale_rule(rule: str) -> None:
    """How the casts evaluate ``clamp(amax, EPS) / 448`` (lingua/float8.py:44): ``"divide"`` (default) is the correctly
    rounded fp32 quotient, what ATen's CPU kernel computes; ``"times_inverse"`` is amax * fp32(1/448), what ATen's GPU
    kernel computes for a division by a Python scalar, i.e. the reference's scales when it runs on a GPU.  Process-wide;
    applies to casts launched after the call."""
    if rule not in SCALE_RULES:
        raise RuntimeError(f"unknown scale rule {rule!r}; known: {sorted(SCALE_RULES)}")
    _lib.check(_lib.load().l8_set_scale_rule(SCALE_RULES[rule]), "l8_set_scale_rule")


def get_scale_rule() -> str:
    code = _lib.load().l8_get_scale_rule()
    return next(name for name, c in SCALE_RULES.items() if c == code)


def gemm_algos() -> Tuple[str, ...]:
    lib = _lib.load()
    return tuple(lib.l8_gemm_algo_name(i + 1).decode() for i in range(lib.l8_gemm_algo_count()))


def _swiglu_ws(R: int, C: int, device, halves: int):
    ws_bytes = _lib.load().l8_swiglu_workspace(R, C) // 2 * halves
    return (torch.empty(ws_bytes, dtype=torch.uint8, device=device) if ws_bytes else None), ws_bytes


def swiglu_cast_rowwise(h1: torch.Tensor, h3: torch.Tensor, want_h: bool = True, col_amax: Optional[torch.Tensor] = None):
    """h = bf16(bf16(silu(h1)) * h3) and its row-wise cast in one pass.
    Returns (h [R,C] bf16 | None, q [R,C] fp8, scale [R,1] fp32, amax [R,1] bf16); ``col_amax`` as in cast_rowwise."""
    h1 = _rows_2d(h1, torch.bfloat16, "swiglu_cast_rowwise(h1)")
    h3 = _rows_2d(h3, torch.bfloat16, "swiglu_cast_rowwise(h3)")
    if h1.shape != h3.shape or h1.device != h3.device:
        raise RuntimeError(f"swiglu_cast_rowwise: h1 {tuple(h1.shape)} and h3 {tuple(h3.shape)} must match")
    st = _prep(h1, "swiglu_cast_rowwise")
    R, C = h1.shape
    dev = h1.device
    h = torch.empty((R, C), dtype=torch.bfloat16, device=dev) if want_h else None
    q = torch.empty((R, C), dtype=torch.float8_e4m3fn, device=dev)
    scale = torch.empty((R, 1), dtype=torch.float32, device=dev)
    amax = torch.empty((R, 1), dtype=torch.bfloat16, device=dev)
    if col_amax is not None and (col_amax.dtype != torch.float32 or col_amax.numel() != C or not col_amax.is_contiguous()):
        raise RuntimeError("swiglu_cast_rowwise: col_amax must be a contiguous fp32 tensor with C elements")
    ws, ws_bytes = _swiglu_ws(R, C, dev, 1) if col_amax is not None else (None, 0)
    with _timed("swiglu_cast_rowwise", R * C * (5 + (2 if want_h else 0)) + 4 * R, dev):
        code = _lib.load().l8_swiglu_cast_rowwise(
            h1.data_ptr(), h3.data_ptr(), R, C, _ld(h1), _ld(h3), h.data_ptr() if want_h else None, C, q.data_ptr(), C,
            scale.data_ptr(), amax.data_ptr(), col_amax.data_ptr() if col_amax is not None else None,
            ws.data_ptr() if ws is not None else None, ws_bytes, st)
    _lib.check(code, "l8_swiglu_cast_rowwise")
    return h, q, scale, amax


def swiglu_bwd_cast_rowwise(dh: torch.Tensor, h1: torch.Tensor, h3: torch.Tensor,
                            col_amax1: Optional[torch.Tensor] = None, col_amax3: Optional[torch.Tensor] = None):
    """Gradients of the SwiGLU gate and their row-wise casts in one pass.
    Returns (g1, g3 [R,C] bf16, q1, q3 [R,C] fp8, scale1, scale3 [R,1] fp32)."""
    dh = _rows_2d(dh, torch.bfloat16, "swiglu_bwd_cast_rowwise(dh)")
    h1 = _rows_2d(h1, torch.bfloat16, "swiglu_bwd_cast_rowwise(h1)")
    h3 = _rows_2d(h3, torch.bfloat16, "swiglu_bwd_cast_rowwise(h3)")
    if not (dh.shape == h1.shape == h3.shape) or not (dh.device == h1.device == h3.device):
        raise RuntimeError("swiglu_bwd_cast_rowwise: dh, h1 and h3 must have the same shape and device")
    if (col_amax1 is None) != (col_amax3 is None):
        raise RuntimeError("swiglu_bwd_cast_rowwise: pass both column amaxes or neither")
    st = _prep(dh, "swiglu_bwd_cast_rowwise")
    R, C = dh.shape
    dev = dh.device
    for ca in (col_amax1, col_amax3):
        if ca is not None and (ca.dtype != torch.float32 or ca.numel() != C or not ca.is_contiguous()):
            raise RuntimeError("swiglu_bwd_cast_rowwise: column amaxes must be contiguous fp32 tensors with C elements")
    g1 = torch.empty((R, C), dtype=torch.bfloat16, device=dev)
    g3 = torch.empty((R, C), dtype=torch.bfloat16, device=dev)
    q1 = torch.empty((R, C), dtype=torch.float8_e4m3fn, device=dev)
    q3 = torch.empty((R, C), dtype=torch.float8_e4m3fn, device=dev)
    s1 = torch.empty((R, 1), dtype=torch.float32, device=dev)
    s3 = torch.empty((R, 1), dtype=torch.float32, device=dev)
    ws, ws_bytes = _swiglu_ws(R, C, dev, 2) if col_amax1 is not None else (None, 0)
    with _timed("swiglu_bwd_cast_rowwise", R * C * 12 + 8 * R, dev):
        code = _lib.load().l8_swiglu_bwd_cast_rowwise(
            dh.data_ptr(), h1.data_ptr(), h3.data_ptr(), R, C, _ld(dh), _ld(h1), _ld(h3), g1.data_ptr(), g3.data_ptr(), C,
            q1.data_ptr(), q3.data_ptr(), C, s1.data_ptr(), s3.data_ptr(),
            col_amax1.data_ptr() if col_amax1 is not None else None, col_amax3.data_ptr() if col_amax3 is not None else None,
            ws.data_ptr() if ws is not None else None, ws_bytes, st)
    _lib.check(code, "l8_swiglu_bwd_cast_rowwise")
    return g1, g3, q1, q3, s1, s3


def rmsnorm_cast_rowwise(x: torch.Tensor, weight: torch.Tensor, eps: float, want_q: bool = True,
                         col_amax: Optional[torch.Tensor] = None, want_rstd: bool = True):
    """y = bf16((f32(x) * rsqrt(mean(x^2) + eps)) * f32(weight)) and its row-wise cast in one pass.
    Returns (y [R,C] bf16, q [R,C] fp8 | None, scale [R,1] fp32 | None, rstd [R,1] fp32 | None)."""
    x = _rows_2d(x, torch.bfloat16, "rmsnorm_cast_rowwise")
    st = _prep(x, "rmsnorm_cast_rowwise")
    R, C = x.shape
    dev = x.device
    if weight.dtype not in (torch.bfloat16, torch.float32) or weight.numel() != C or weight.device != dev:
        raise RuntimeError("rmsnorm_cast_rowwise: weight must be bf16 or fp32 with C elements on the same device")
    weight = weight.contiguous()
    if col_amax is not None and (not want_q or col_amax.dtype != torch.float32 or col_amax.numel() != C or not col_amax.is_contiguous()):
        raise RuntimeError("rmsnorm_cast_rowwise: col_amax needs the cast and must be a contiguous fp32 tensor with C elements")
    y = torch.empty((R, C), dtype=torch.bfloat16, device=dev)
    q = torch.empty((R, C), dtype=torch.float8_e4m3fn, device=dev) if want_q else None
    scale = torch.empty((R, 1), dtype=torch.float32, device=dev) if want_q else None
    rstd = torch.empty((R, 1), dtype=torch.float32, device=dev) if want_rstd else None
    ws, ws_bytes = None, 0
    if col_amax is not None:
        ws_bytes = _lib.load().l8_rmsnorm_workspace(R, C)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev) if ws_bytes else None
    with _timed("rmsnorm_cast_rowwise", R * C * (4 + (1 if want_q else 0)) + 8 * R, dev):
        code = _lib.load().l8_rmsnorm_cast_rowwise(
            x.data_ptr(), weight.data_ptr(), int(weight.dtype == torch.float32), R, C, _ld(x), float(eps), y.data_ptr(), C,
            q.data_ptr() if want_q else None, C, scale.data_ptr() if want_q else None,
            rstd.data_ptr() if want_rstd else None, col_amax.data_ptr() if col_amax is not None else None,
            ws.data_ptr() if ws is not None else None, ws_bytes, st)
    _lib.check(code, "l8_rmsnorm_cast_rowwise")
    return y, q, scale, rstd


def rmsnorm_bwd(gy: torch.Tensor, x: torch.Tensor, weight: torch.Tensor, rstd: torch.Tensor):
    """Backward of the RMSNorm: returns (gx [R,C] bf16, gw [C] fp32) from gy, x (bf16 [R,C]), weight [C], rstd [R,1] fp32."""
    gy = _rows_2d(gy, torch.bfloat16, "rmsnorm_bwd(gy)")
    x = _rows_2d(x, torch.bfloat16, "rmsnorm_bwd(x)")
    if gy.shape != x.shape or gy.device != x.device:
        raise RuntimeError("rmsnorm_bwd: gy and x must have the same shape and device")
    st = _prep(x, "rmsnorm_bwd")
    R, C = x.shape
    dev = x.device
    if weight.dtype not in (torch.bfloat16, torch.float32) or weight.numel() != C or weight.device != dev:
        raise RuntimeError("rmsnorm_bwd: weight must be bf16 or fp32 with C elements on the same device")
    if rstd.dtype != torch.float32 or rstd.numel() != R or rstd.device != dev:
        raise RuntimeError("rmsnorm_bwd: rstd must be fp32 with R elements on the same device")
    weight, rstd = weight.contiguous(), rstd.contiguous()
    gx = torch.empty((R, C), dtype=torch.bfloat16, device=dev)
    gw = torch.empty((C,), dtype=torch.float32, device=dev)
    ws_bytes = _lib.load().l8_rmsnorm_bwd_workspace(R, C)
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    with _timed("rmsnorm_bwd", R * C * 6 + 4 * R, dev):
        code = _lib.load().l8_rmsnorm_bwd(gy.data_ptr(), x.data_ptr(), weight.data_ptr(), int(weight.dtype == torch.float32),
                                          rstd.data_ptr(), R, C, _ld(gy), _ld(x), gx.data_ptr(), C, gw.data_ptr(),
                                          ws.data_ptr(), ws_bytes, st)
    _lib.check(code, "l8_rmsnorm_bwd")
    return gx, gw
