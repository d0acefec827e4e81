"""One product for the attention projections.

The reference's attention applies three linears to the same activation
(lingua/transformer.py:357-359: ``xq = self.wq(x)``, ``xk = self.wk(x)``,
``xv = self.wv(x)``).  Converted by ``convert_linears_to_fp8`` they already
share one quantised copy of ``x``; ``fuse_qkv`` additionally makes their three
forward products one: the three weights are quantised row-wise straight into
one ``[Nq+Nk+Nv, K]`` operand (no concatenation pass: the cast kernels write
into row slices of it) and a single GEMM produces ``[T, Nq+Nk+Nv]``, of which
the three linears return column slices.  Same recipe, same scales (every weight
row keeps its own), so the same bits as three separate products.

Backward stays per linear (lingua/float8.py:99-131): the three dgrads have
different row scales and cannot be one product; the three wgrads share the
token-dimension copy of ``x`` through the memo of ``lingua_amd.float8``.

Nothing changes in the attention module or in the state dict: ``wq`` computes
all three products when it is called and keeps the other two for ``wk`` and
``wv``, which hand them out when they are called on the same activation (and
fall back to their own product otherwise).  Opt-in: ``fuse_qkv(model)`` after
``convert_linears_to_fp8``.
"""
import re

import torch

from . import float8 as f8
from . import ops


class Fp8QKVFn(torch.autograd.Function):
    """``(x @ wq.T, x @ wk.T, x @ wv.T)`` as one fp8 product; x [T,K], weights [N_i,K], no biases."""

    @staticmethod
    def forward(ctx, x, wq, wk, wv):
        ws = (wq, wk, wv)
        for t in (x,) + ws:
            if t.dtype != torch.bfloat16:
                raise RuntimeError(f"Fp8QKVFn: bf16 input and weights required, got {t.dtype}")
        cfg = f8.config
        need_stats = cfg.fp8_wgrad and any(w.requires_grad for w in ws)
        f8._bwd_cast.clear(x)
        hit = f8._fwd_cast.get(x, ("qkv", wq.data_ptr())) if cfg.share_input_casts else None
        if hit is not None and (hit[2] is not None or not need_stats):
            qx, sx, x_col = hit
            if not need_stats:
                x_col = None
        else:
            x_col = torch.empty(x.shape[1], dtype=torch.float32, device=x.device) if need_stats else None
            qx, sx, _ = ops.cast_rowwise(x, col_amax=x_col)
            if cfg.share_input_casts:
                f8._fwd_cast.put(x, (qx, sx, x_col), ("qkv", wq.data_ptr()))
        K = x.shape[1]
        sizes = [w.shape[0] for w in ws]
        qw = torch.empty((sum(sizes), K), dtype=torch.float8_e4m3fn, device=x.device)
        sw = torch.empty((sum(sizes), 1), dtype=torch.float32, device=x.device)
        amaxes, o = [], 0
        for w, n in zip(ws, sizes):
            _, _, amax_w = ops.cast_rowwise(w, out_q=qw[o:o + n], out_scale=sw[o:o + n])
            amaxes.append(amax_w)
            o += n
        y = ops.gemm_nt(qx, qw, sx, sw, None, algo=cfg.gemm_algo)
        ctx.fp8_wgrad, ctx.gemm_algo, ctx.has_col = cfg.fp8_wgrad, cfg.gemm_algo, x_col is not None
        ctx.need = (x.requires_grad,) + tuple(w.requires_grad for w in ws)
        ctx.save_for_backward(x, *ws, *amaxes, *([x_col] if x_col is not None else []))
        outs, o = [], 0
        for n in sizes:
            outs.append(y[:, o:o + n])
            o += n
        return tuple(outs)

    @staticmethod
    def backward(ctx, *grads):
        saved = ctx.saved_tensors
        x, ws, amaxes = saved[0], saved[1:4], saved[4:7]
        x_col = saved[7] if ctx.has_col else None
        gx, gws = None, [None, None, None]
        for i, g in enumerate(grads):
            if g is None or not (ctx.need[0] or ctx.need[1 + i]):
                continue
            ga, gb, _ = f8.linear_backward(g.contiguous(), x, ws[i], amaxes[i], x_col, ctx.need[0], ctx.need[1 + i], False,
                                           ctx.fp8_wgrad, ctx.gemm_algo)
            gws[i] = gb
            if ga is not None:
                gx = ga if gx is None else gx.add_(ga)
        return (gx, *gws)


class _QKVGroup:
    """What ``wq`` computed for ``wk`` and ``wv``: handed out once each, to a call on the same activation."""

    def __init__(self):
        self.key = None
        self.pending = {}

    @staticmethod
    def key_of(x):
        return (x.data_ptr(), tuple(x.shape), tuple(x.stride()), x._version, torch.is_grad_enabled())


class Fp8QKVLinear(f8.Fp8Linear):
    """An ``Fp8Linear`` that is one of the three attention projections of a ``fuse_qkv`` group."""

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        group, role = self._qkv_group, self._qkv_role
        x = input.flatten(end_dim=-2)
        if x.is_inference() or f8.config.use_custom_ops:
            return super().forward(input)
        key = group.key_of(x)
        if role == 0:
            q, k, v = Fp8QKVFn.apply(x, *(lin.weight for lin in self._qkv_members()))
            group.key, group.pending = key, {1: k, 2: v}
            out = q
        else:
            out = group.pending.pop(role, None) if group.key == key else None
            if out is None:
                return super().forward(input)
        return out.unflatten(0, input.shape[:-1])

    def _qkv_members(self):
        return self._qkv_group.members


def fuse_qkv(root_module: torch.nn.Module, filter: str = r"attention$") -> torch.nn.Module:
    """In every module whose dotted name matches ``filter`` and that has bias-free ``Fp8Linear`` children ``wq``,
    ``wk``, ``wv`` over the same input width (the reference's Attention, lingua/transformer.py:325-359), make the
    three forward products one.  The caller vouches that the module applies ``wq`` first and all three to the same
    tensor; anything else still computes the right thing, one product at a time."""
    filter_re = re.compile(filter)
    for name, module in root_module.named_modules():
        if not filter_re.search(name):
            continue
        lins = [getattr(module, n, None) for n in ("wq", "wk", "wv")]
        if any(isinstance(l, Fp8QKVLinear) for l in lins):
            continue
        if not all(type(l) is f8.Fp8Linear and l.bias is None for l in lins) or len({l.in_features for l in lins}) != 1:
            raise RuntimeError(f"fuse_qkv: {name!r} has no bias-free Fp8Linear children wq, wk, wv of one input width "
                               "(run convert_linears_to_fp8 first)")
        group = _QKVGroup()
        group.members = tuple(lins)
        for role, lin in enumerate(lins):
            lin.__class__ = Fp8QKVLinear
            object.__setattr__(lin, "_qkv_group", group)
            object.__setattr__(lin, "_qkv_role", role)
    return root_module
