"""SwiGLU MLP with the float8 recipe applied to its three linears and the gate
fused into the casts on either side of it.

The reference's MLP is ``w2(F.silu(w1(x)) * w3(x))`` (lingua/transformer.py:430-471)
with ``w1 / w2 / w3`` turned into ``Fp8Linear`` by ``convert_linears_to_fp8``
(lingua/float8.py:150-191).  Run that way, every linear quantises its own
input and the gate is three bf16 elementwise kernels in forward and three in
backward.  ``Fp8FeedForward`` computes the same function with the same
quantisation recipe (``lingua_amd.float8``), but

  * ``x`` is quantised once for ``w1`` and ``w3`` (forward) and once, along
    the token dimension, for their two wgrads (backward);
  * the gate and the cast of the ``w2`` input are one kernel
    (``l8_swiglu_cast_rowwise``), the gate's backward and the casts of its two
    gradients another (``l8_swiglu_bwd_cast_rowwise``).

It is opt-in: ``fuse_feed_forward(model)`` swaps modules that look like the
reference's ``FeedForward`` after (or instead of) ``convert_linears_to_fp8``.
"""
import re
from typing import Optional

import torch

from . import float8 as f8
from . import ops


class Fp8SwiGLUFn(torch.autograd.Function):
    """``y = (silu(x @ w1.T) * (x @ w3.T)) @ w2.T`` with fp8 operands, x [T,D], w1/w3 [F,D], w2 [D,F]."""

    @staticmethod
    def forward(ctx, x, w1, w3, w2):
        for t in (x, w1, w3, w2):
            if t.dtype != torch.bfloat16:
                raise RuntimeError(f"Fp8SwiGLUFn: bf16 input and weights required, got {t.dtype}")
        cfg = f8.config
        fp8_wgrad = cfg.fp8_wgrad
        algo = cfg.gemm_algo
        need_x_col = fp8_wgrad and (w1.requires_grad or w3.requires_grad)
        # an Fp8RMSNorm in front of this block has filed its output already quantised (with its column amaxes when
        # it ran in training mode): take that copy instead of quantising the activation a second time
        hit = f8._fwd_cast.get(x, ("swiglu", w1.data_ptr())) if cfg.share_input_casts else None
        if hit is not None and (hit[2] is not None or not need_x_col):
            qx, sx, x_col = hit
            if not need_x_col:
                x_col = None
        else:
            x_col = torch.empty(x.shape[1], dtype=torch.float32, device=x.device) if need_x_col else None
            qx, sx, _ = ops.cast_rowwise(x, col_amax=x_col)
        q1, s1, amax_w1 = f8.weight_cast_rowwise(w1)
        q3, s3, amax_w3 = f8.weight_cast_rowwise(w3)
        h1 = ops.gemm_nt(qx, q1, sx, s1, None, algo=algo)
        h3 = ops.gemm_nt(qx, q3, sx, s3, None, algo=algo)
        del qx, q1, q3
        h_col = torch.empty(w2.shape[1], dtype=torch.float32, device=x.device) if fp8_wgrad and w2.requires_grad else None
        h, qh, sh, _ = ops.swiglu_cast_rowwise(h1, h3, want_h=w2.requires_grad, col_amax=h_col)
        q2, s2, amax_w2 = f8.weight_cast_rowwise(w2)
        y = ops.gemm_nt(qh, q2, sh, s2, None, algo=algo)

        ctx.fp8_wgrad, ctx.gemm_algo = fp8_wgrad, algo
        ctx.need = (x.requires_grad, w1.requires_grad, w3.requires_grad, w2.requires_grad)
        ctx.opt = (h is not None, x_col is not None, h_col is not None)
        saved = [x, w1, w3, w2, h1, h3, amax_w1, amax_w3, amax_w2]
        saved += [t for t in (h, x_col, h_col) if t is not None]
        ctx.save_for_backward(*saved)
        return y

    @staticmethod
    def backward(ctx, gy):
        if gy.dtype != torch.bfloat16:
            raise RuntimeError(f"Fp8SwiGLUFn.backward: bf16 grad_out required, got {gy.dtype}")
        saved = list(ctx.saved_tensors)
        x, w1, w3, w2, h1, h3, amax_w1, amax_w3, amax_w2 = saved[:9]
        rest = saved[9:]
        h = rest.pop(0) if ctx.opt[0] else None
        x_col = rest.pop(0) if ctx.opt[1] else None
        h_col = rest.pop(0) if ctx.opt[2] else None
        need_x, need_w1, need_w3, need_w2 = ctx.need
        fp8_wgrad, algo = ctx.fp8_wgrad, ctx.gemm_algo
        dev = gy.device
        D, F = w1.shape[1], w1.shape[0]

        gx = gw1 = gw3 = gw2 = None
        if not (need_x or need_w1 or need_w3):
            # only w2 learns: its wgrad needs neither dh nor the gate's backward
            if need_w2:
                gw2 = _wgrad(gy, None, h, h_col, fp8_wgrad, algo)
            return gx, gw1, gw3, gw2

        gy_col = torch.empty(D, dtype=torch.float32, device=dev) if fp8_wgrad and need_w2 else None
        qgy, sgy, _ = ops.cast_rowwise(gy, col_amax=gy_col)
        qw2t, sw2t = f8.weight_cast_tensorwise_t(w2, amax_w2)
        dh = ops.gemm_nt(qgy, qw2t, sgy, sw2t, None, algo=algo)
        del qgy, qw2t
        if need_w2:
            gw2 = _wgrad(gy, gy_col, h, h_col, fp8_wgrad, algo)

        want_cols = fp8_wgrad and (need_w1 or need_w3)
        g1_col = torch.empty(F, dtype=torch.float32, device=dev) if want_cols else None
        g3_col = torch.empty(F, dtype=torch.float32, device=dev) if want_cols else None
        g1, g3, qg1, qg3, sg1, sg3 = ops.swiglu_bwd_cast_rowwise(dh, h1, h3, g1_col, g3_col)
        del dh
        if need_x:
            qw1t, sw1t = f8.weight_cast_tensorwise_t(w1, amax_w1)
            gx = ops.gemm_nt(qg1, qw1t, sg1, sw1t, None, algo=algo)
            qw3t, sw3t = f8.weight_cast_tensorwise_t(w3, amax_w3)
            gx += ops.gemm_nt(qg3, qw3t, sg3, sw3t, None, algo=algo)
        del qg1, qg3
        if need_w1 or need_w3:
            if fp8_wgrad:
                if x_col is None:
                    x_col = ops.col_amax(x)
                qxt, sxt = ops.cast_colwise_transposed(x, x_col)   # shared by both wgrads
                if need_w1:
                    qgt, sgt = ops.cast_colwise_transposed(g1, g1_col)
                    gw1 = ops.gemm_nt(qgt, qxt, sgt, sxt, None, algo=algo)
                if need_w3:
                    qgt, sgt = ops.cast_colwise_transposed(g3, g3_col)
                    gw3 = ops.gemm_nt(qgt, qxt, sgt, sxt, None, algo=algo)
            else:
                gw1 = g1.t() @ x if need_w1 else None
                gw3 = g3.t() @ x if need_w3 else None
        return gx, gw1, gw3, gw2


def _wgrad(g, g_col, a, a_col, fp8_wgrad, algo):
    """dW = g.T @ a, fp8 with token-dimension scales or bf16 (lingua/float8.py:123)."""
    if not fp8_wgrad:
        return g.t() @ a
    if g_col is None:
        g_col = ops.col_amax(g)
    if a_col is None:
        a_col = ops.col_amax(a)
    qgt, sgt = ops.cast_colwise_transposed(g, g_col)
    qat, sat = ops.cast_colwise_transposed(a, a_col)
    return ops.gemm_nt(qgt, qat, sgt, sat, None, algo=algo)


class Fp8FeedForward(torch.nn.Module):
    """Stands in for a module computing ``w2(silu(w1(x)) * w3(x))``; keeps the three
    linears as children under their names, so parameters and state-dict keys do not change."""

    def __init__(self, w1: torch.nn.Linear, w3: torch.nn.Linear, w2: torch.nn.Linear):
        super().__init__()
        for lin in (w1, w3, w2):
            if not isinstance(lin, torch.nn.Linear) or lin.bias is not None:
                raise RuntimeError("Fp8FeedForward: w1, w3 and w2 must be bias-free nn.Linear modules")
        if w1.weight.shape != w3.weight.shape or w2.weight.shape != w1.weight.shape[::-1]:
            raise RuntimeError(
                f"Fp8FeedForward: inconsistent shapes w1 {tuple(w1.weight.shape)}, w3 {tuple(w3.weight.shape)}, "
                f"w2 {tuple(w2.weight.shape)}")
        self.w1, self.w3, self.w2 = w1, w3, w2

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = Fp8SwiGLUFn.apply(x.flatten(end_dim=-2), self.w1.weight, self.w3.weight, self.w2.weight)
        return y.unflatten(0, x.shape[:-1])


def fuse_feed_forward(root_module: torch.nn.Module, filter: str = r"feed_forward$") -> torch.nn.Module:
    """Swap every module whose dotted name matches ``filter`` and whose children are exactly the
    bias-free linears ``w1``, ``w2``, ``w3`` (the reference's FeedForward, lingua/transformer.py:430-471)
    for an ``Fp8FeedForward`` over the same linears.  The caller vouches that the module computes
    ``w2(silu(w1(x)) * w3(x))``; a matching module of any other shape raises."""
    filter_re = re.compile(filter)

    def replace(module: torch.nn.Module, name: str) -> torch.nn.Module:
        if isinstance(module, Fp8FeedForward) or not filter_re.search(name):
            return module
        children = dict(module.named_children())
        if set(children) != {"w1", "w2", "w3"} or list(module.parameters(recurse=False)):
            raise RuntimeError(f"fuse_feed_forward: {name!r} ({type(module).__name__}) is not a w1/w2/w3 SwiGLU block")
        return Fp8FeedForward(children["w1"], children["w3"], children["w2"])

    return f8.named_replace(replace, root_module)
