"""The row-wise float8 recipe as a chain of PyTorch CPU ops -- TEST INFRASTRUCTURE ONLY.

Second, independent restatement of the reference algorithm (the first is the
integer C code in ``fp8_recipe_oracle.c``).  Every function issues the same
ATen ops, in the same order and dtypes, as the cited reference lines, with one
deliberate difference: ``torch._scaled_mm`` with row-wise scales does not exist
on CPU, so the product is "dequantise, fp32 matmul, round to bf16", which is
the definition of the expected output that the benchmark spec gives.

This module is also what the benchmark times as ``cpu_baseline`` (kind "port").
"""
import torch

EPS = 1e-12  # lingua/float8.py:11
E4M3_MAX = torch.finfo(torch.float8_e4m3fn).max  # 448.0
# ATen's GPU kernel divides a tensor by a Python scalar by multiplying with the scalar's fp32 reciprocal; its CPU
# kernel divides.  True makes scale() on CPU tensors do what the GPU kernel does (oracle.scale_rule sets this).
SCALE_TIMES_INVERSE = False


def row_amax(t: torch.Tensor) -> torch.Tensor:
    """lingua/float8.py:86 with splitk == 1: [R,C] -> [R,1], same dtype as t."""
    return t.abs().unflatten(-1, (1, -1)).amax(dim=-1)


def tensor_amax_from_rows(amax_rows: torch.Tensor, n_rows_out: int) -> torch.Tensor:
    """lingua/float8.py:115-118: [N,1] row amaxes -> [n_rows_out,1], all equal to the tensor amax."""
    a = amax_rows.t().unflatten(-1, (1, -1)).amax(dim=-1)
    return a.repeat_interleave(n_rows_out // a.shape[0], dim=0, output_size=n_rows_out)


def tile_broadcast(b: torch.Tensor, shape) -> torch.Tensor:
    """lingua/float8.py:24-30 as an expansion: b [m,n] -> [R,C] where element (r,c) is b[r // (R/m), c // (C/n)],
    i.e. the operand is cut into m x n equal chunks and each chunk sees one element of b."""
    R, C = shape
    m, n = b.shape
    return b.repeat_interleave(R // m, dim=0).repeat_interleave(C // n, dim=1)


def scale(t: torch.Tensor, amax_t: torch.Tensor):
    """lingua/float8.py:43-47.  amax_t is [R,1] (row-wise), [1,1] (tensor-wise) or [R,g] (g column groups per row)."""
    if SCALE_TIMES_INVERSE and not amax_t.is_cuda:
        scale_t = torch.clamp(amax_t.float(), min=EPS) * (torch.ones((), dtype=torch.float32) / E4M3_MAX)
    else:
        scale_t = torch.clamp(amax_t.float(), min=EPS) / E4M3_MAX
    recip = scale_t.reciprocal()
    t_fp8 = (t * tile_broadcast(recip, t.shape)).to(torch.float8_e4m3fn)
    return t_fp8, scale_t


def subrow_amax(t: torch.Tensor, g: int) -> torch.Tensor:
    """lingua/float8.py:86 with splitk == g: [R,C] -> [R,g] amax of each of the g column groups of a row."""
    return t.abs().unflatten(-1, (g, -1)).amax(dim=-1)


def dequant_matmul(q1, s1, q2_t, s2_t, bias=None) -> torch.Tensor:
    """bf16( (q1*s1) @ (q2_t*s2_t)^T + bias ), fp32 throughout.  With g > 1 scale columns the result is the
    fp32 sum of the g per-group products, each rounded to bf16 first (one rank's output under tensor
    parallelism, lingua/float8.py:14-21 and :65-77), rounded to bf16 once more."""
    g = s1.shape[1]
    if g == 1 and s2_t.shape[1] == 1:
        res = (q1.float() * s1) @ (q2_t.float() * s2_t).t()
        if bias is not None:
            res = res + bias.float()
        return res.to(torch.bfloat16)
    assert s2_t.shape[1] == g
    cs = q1.shape[1] // g
    acc = torch.zeros((q1.shape[0], q2_t.shape[0]), dtype=torch.float32)
    for j in range(g):
        sl = slice(j * cs, (j + 1) * cs)
        acc += dequant_matmul(q1[:, sl], s1[:, j:j + 1], q2_t[:, sl], s2_t[:, j:j + 1], bias if j == 0 else None).float()
    return acc.to(torch.bfloat16)


def matmul(first, amax_first, second_t, amax_second_t, bias=None) -> torch.Tensor:
    """lingua/float8.py:50-79 (operand roles: both reduction-contiguous)."""
    q1, s1 = scale(first, amax_first)
    q2, s2 = scale(second_t, amax_second_t)
    return dequant_matmul(q1, s1, q2, s2, bias)


def linear_forward(a, b_t, bias=None):
    """lingua/float8.py:85-88"""
    return matmul(a, row_amax(a), b_t, row_amax(b_t), bias)


def linear_dgrad(grad_out, b_t):
    """lingua/float8.py:110-119"""
    amax_b_t = row_amax(b_t)
    b = b_t.t().contiguous()
    amax_b = tensor_amax_from_rows(amax_b_t, b.shape[0])
    return matmul(grad_out, row_amax(grad_out), b, amax_b)


def linear_wgrad_bf16(grad_out, a):
    """lingua/float8.py:123"""
    return grad_out.t() @ a


def linear_wgrad_fp8(grad_out, a):
    """fp8 wgrad (not in the reference): the recipe's scale() applied to the
    operands transposed so that the token dimension is the reduction one."""
    gt = grad_out.t().contiguous()
    at = a.t().contiguous()
    return matmul(gt, row_amax(gt), at, row_amax(at))


def linear_fwd_bwd(a, b_t, grad_out, bias=None, wgrad_fp8=True):
    out = linear_forward(a, b_t, bias)
    grad_a = linear_dgrad(grad_out, b_t)
    grad_b = linear_wgrad_fp8(grad_out, a) if wgrad_fp8 else linear_wgrad_bf16(grad_out, a)
    grad_bias = grad_out.sum(dim=0) if bias is not None else None  # lingua/float8.py:127
    return out, grad_a, grad_b, grad_bias


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """lingua/transformer.py:283-289: ``_norm(x.float()) * weight.float()`` cast back to x's dtype."""
    xf = x.float()
    out = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
    return (out * weight.float()).type_as(x)


def swiglu_gate(h1: torch.Tensor, h3: torch.Tensor) -> torch.Tensor:
    """lingua/transformer.py:469-471 between the linears: ``F.silu(h1) * h3`` as eager
    PyTorch runs it on bf16 tensors (silu in fp32 rounded to bf16, then a bf16 multiply)."""
    return torch.nn.functional.silu(h1) * h3


def swiglu_gate_bwd(dh: torch.Tensor, h1: torch.Tensor, h3: torch.Tensor):
    """Gradients of ``swiglu_gate`` w.r.t. h1 and h3 as autograd produces them (bf16
    mul backward twice, silu_backward in fp32 rounded to bf16)."""
    a = h1.detach().clone().requires_grad_(True)
    b = h3.detach().clone().requires_grad_(True)
    swiglu_gate(a, b).backward(dh)
    return a.grad, b.grad


def swiglu_mlp_fwd_bwd(x, w1, w2, w3, grad_y):
    """SwiGLU MLP of lingua/transformer.py:469-471 with every linear in fp8,
    forward and backward; elementwise work in bf16 as eager PyTorch does it."""
    x1 = linear_forward(x, w1)
    x3 = linear_forward(x, w3)
    h = torch.nn.functional.silu(x1) * x3
    y = linear_forward(h, w2)
    # backward
    dh = linear_dgrad(grad_y, w2)
    dw2 = linear_wgrad_fp8(grad_y, h)
    x1f, x3f, dhf = x1.float(), x3.float(), dh.float()
    sig = torch.sigmoid(x1f)
    dx3 = (dhf * (x1f * sig)).to(torch.bfloat16)
    dx1 = (dhf * x3f * (sig * (1 + x1f * (1 - sig)))).to(torch.bfloat16)
    dx = (linear_dgrad(dx1, w1).float() + linear_dgrad(dx3, w3).float()).to(torch.bfloat16)
    dw1 = linear_wgrad_fp8(dx1, x)
    dw3 = linear_wgrad_fp8(dx3, x)
    return y, dx, dw1, dw2, dw3
