"""RMSNorm whose output arrives at the fp8 linears already quantised.

``Fp8RMSNorm`` is a drop-in for the reference's ``RMSNorm``
(lingua/transformer.py:264-292: ``(x.float() * rsqrt(mean(x^2) + eps) * weight.float()).type_as(x)``).
Its backward is one kernel too (``l8_rmsnorm_bwd``).  Its forward (``l8_rmsnorm_cast_rowwise``) writes the bf16
output and, from the same registers, the row-wise fp8 copy that the linears
fed by the norm (wq / wk / wv, w1 / w3) would otherwise each compute in a pass
of their own (lingua/float8.py:86-87, :43-47).  The quantised copy is handed
over through the memo of ``lingua_amd.float8`` that already lets such linears
share one cast, so nothing changes in the attention / MLP modules.

Opt-in: ``fuse_rmsnorm(model)`` after (or before) ``convert_linears_to_fp8``.
"""
import re

import torch

from . import float8 as f8
from . import ops


class Fp8RMSNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, eps, training):
        if x.dtype != torch.bfloat16:
            raise RuntimeError(f"Fp8RMSNorm: bf16 activations required, got {x.dtype}")
        x2d = x.flatten(end_dim=-2)
        col = torch.empty(x2d.shape[1], dtype=torch.float32, device=x.device) if (training and f8.config.fp8_wgrad) else None
        y2d, q, s, rstd = ops.rmsnorm_cast_rowwise(x2d, weight, eps, want_q=True, col_amax=col, want_rstd=True)
        if f8.config.share_input_casts:
            f8._fwd_cast.put(y2d, (q, s, col), "rmsnorm")
        ctx.save_for_backward(x2d, weight, rstd)
        ctx.x_shape = x.shape
        return y2d.unflatten(0, x.shape[:-1])

    @staticmethod
    def backward(ctx, gy):
        x2d, weight, rstd = ctx.saved_tensors
        if gy.dtype != torch.bfloat16:
            raise RuntimeError(f"Fp8RMSNorm.backward: bf16 grad_out required, got {gy.dtype}")
        gx2d, gw = ops.rmsnorm_bwd(gy.flatten(end_dim=-2), x2d, weight, rstd)
        gx = gx2d.reshape(ctx.x_shape) if ctx.needs_input_grad[0] else None
        return gx, (gw.to(weight.dtype) if ctx.needs_input_grad[1] else None), None, None


class Fp8RMSNorm(torch.nn.Module):
    """Same parameters and state-dict keys as the reference's RMSNorm (``weight``; ``eps`` attribute)."""

    def __init__(self, dim: int, eps: float = 1e-6, weight: torch.nn.Parameter = None):
        super().__init__()
        self.eps = eps
        self.weight = weight if weight is not None else torch.nn.Parameter(torch.ones(dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # grad mode is read here: inside an autograd Function's forward it is always off
        return Fp8RMSNormFn.apply(x, self.weight, self.eps, torch.is_grad_enabled())

    def reset_parameters(self):
        torch.nn.init.ones_(self.weight)


def fuse_rmsnorm(root_module: torch.nn.Module, filter: str = r"(attention_norm|ffn_norm)$") -> torch.nn.Module:
    """Swap every module whose dotted name matches ``filter`` and that looks like the reference's RMSNorm
    (class name ``RMSNorm``, a 1-D ``weight`` and an ``eps``) for an ``Fp8RMSNorm`` over the same Parameter.
    The default filter takes the two norms of a block, whose outputs feed fp8 linears, and leaves the final
    norm in front of the bf16 output head alone."""
    filter_re = re.compile(filter)

    def replace(module: torch.nn.Module, name: str) -> torch.nn.Module:
        if isinstance(module, Fp8RMSNorm) or not filter_re.search(name):
            return module
        w = getattr(module, "weight", None)
        if type(module).__name__ != "RMSNorm" or not isinstance(w, torch.nn.Parameter) or w.dim() != 1 or not hasattr(module, "eps"):
            raise RuntimeError(f"fuse_rmsnorm: {name!r} ({type(module).__name__}) is not an RMSNorm with weight and eps")
        return Fp8RMSNorm(w.numel(), float(module.eps), weight=w)

    return f8.named_replace(replace, root_module)
