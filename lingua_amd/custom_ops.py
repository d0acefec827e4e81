"""The fp8 linear as ``torch.library`` operators.

The reference marks its autograd function ``allow_in_graph`` (lingua/float8.py:82) so that
``model.compile()`` (lingua/distributed.py:476-480) keeps working, and lingua's selective activation
checkpointing decides what to save by operator name (``aten._scaled_mm`` in lingua/distributed.py:43-50).
Both need the path to be visible as operators rather than as Python that calls into a C library:

  ``lingua_amd::fp8_linear_fwd(a, b_t, bias, need_wgrad_stats, algo) -> (out, amax_b_t, a_col_amax)``
  ``lingua_amd::fp8_linear_bwd(grad_out, a, b_t, amax_b_t, a_col_amax, need_a, need_b, need_bias,
                               fp8_wgrad, algo) -> (grad_a, grad_b, grad_bias)``

with fake (shape-only) implementations and an autograd formula tying them together.  ``fp8_linear`` below is
the differentiable entry; ``lingua_amd.float8.config.use_custom_ops = True`` makes ``Fp8Linear`` use it.  A
checkpointing policy that wants the product saved lists ``torch.ops.lingua_amd.fp8_linear_fwd.default``.
Tensors that an invocation does not produce come back with zero elements (operators cannot return None).
"""
from typing import Optional, Tuple

import torch

from . import float8 as f8


def _empty(like: torch.Tensor, dtype=None) -> torch.Tensor:
    return like.new_empty((0,), dtype=dtype or like.dtype)


@torch.library.custom_op("lingua_amd::fp8_linear_fwd", mutates_args=(), device_types="cuda")
def fp8_linear_fwd(a: torch.Tensor, b_t: torch.Tensor, bias: Optional[torch.Tensor], need_wgrad_stats: bool,
                   algo: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    out, amax_b_t, a_col_amax = f8.linear_forward(a, b_t, bias, need_wgrad_stats, algo)
    # the column amaxes may be shared with another linear on the same activation: operators return fresh tensors
    return out, amax_b_t, (a_col_amax.clone() if a_col_amax is not None else _empty(a, torch.float32))


@fp8_linear_fwd.register_fake
def _(a, b_t, bias, need_wgrad_stats, algo):
    return (a.new_empty((a.shape[0], b_t.shape[0])), b_t.new_empty((b_t.shape[0], 1)),
            a.new_empty((a.shape[1] if need_wgrad_stats else 0,), dtype=torch.float32))


@torch.library.custom_op("lingua_amd::fp8_linear_bwd", mutates_args=(), device_types="cuda")
def fp8_linear_bwd(grad_out: torch.Tensor, a: torch.Tensor, b_t: torch.Tensor, amax_b_t: torch.Tensor,
                   a_col_amax: torch.Tensor, need_a: bool, need_b: bool, need_bias: bool, fp8_wgrad: bool,
                   algo: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    ga, gb, gbias = f8.linear_backward(grad_out.contiguous(), a, b_t, amax_b_t,
                                       a_col_amax if a_col_amax.numel() else None, need_a, need_b, need_bias,
                                       fp8_wgrad, algo)
    return (ga if ga is not None else _empty(a), gb if gb is not None else _empty(b_t),
            gbias if gbias is not None else _empty(grad_out))


@fp8_linear_bwd.register_fake
def _(grad_out, a, b_t, amax_b_t, a_col_amax, need_a, need_b, need_bias, fp8_wgrad, algo):
    return (a.new_empty(a.shape if need_a else (0,)), b_t.new_empty(b_t.shape if need_b else (0,)),
            grad_out.new_empty((grad_out.shape[1],) if need_bias else (0,)))


def _setup_context(ctx, inputs, output):
    a, b_t, bias, _, algo = inputs
    _, amax_b_t, a_col_amax = output
    ctx.save_for_backward(a, b_t, amax_b_t, a_col_amax)
    ctx.algo = algo
    ctx.fp8_wgrad = f8.config.fp8_wgrad
    ctx.has_bias = bias is not None


def _backward(ctx, grad_out, _grad_amax, _grad_col):
    a, b_t, amax_b_t, a_col_amax = ctx.saved_tensors
    need_a, need_b = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
    need_bias = ctx.has_bias and ctx.needs_input_grad[2]
    ga, gb, gbias = fp8_linear_bwd(grad_out, a, b_t, amax_b_t, a_col_amax, need_a, need_b, need_bias, ctx.fp8_wgrad, ctx.algo)
    return (ga if need_a else None, gb if need_b else None, gbias if need_bias else None, None, None)


fp8_linear_fwd.register_autograd(_backward, setup_context=_setup_context)


def fp8_linear(a: torch.Tensor, b_t: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """``a @ b_t.T + bias`` in row-wise fp8 through the operators above (2-D ``a``)."""
    need_wgrad_stats = f8.config.fp8_wgrad and b_t.requires_grad and torch.is_grad_enabled()
    return fp8_linear_fwd(a, b_t, bias, need_wgrad_stats, f8.config.gemm_algo)[0]
