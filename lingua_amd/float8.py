"""Drop-in for the float8 linear path of facebookresearch/lingua
(``lingua/float8.py``) on MI355X: same names, arguments and error behaviour,
with every device operation done by the gfx950 kernels in ``liblingua_fp8.so``.

Mirrors
  * ``EPS``                          lingua/float8.py:11
  * ``scale(t, amax_t)``             lingua/float8.py:43-47
  * ``matmul(...)``                  lingua/float8.py:50-79
  * ``Fp8LinearFn``                  lingua/float8.py:82-131
  * ``Fp8Linear``                    lingua/float8.py:134-138
  * ``named_replace``                lingua/float8.py:141-147
  * ``convert_linears_to_fp8``       lingua/float8.py:150-191

Differences, all deliberate:
  * single GPU: the tensor-parallel helpers (``get_splitk``, ``apply_to_partial``
    and the DTensor back-ports, lingua/float8.py:14-40,194-315) are not here;
    ``Fp8LinearFn`` always uses one scale group per row, while ``scale`` and
    ``matmul`` also accept the ``[R,g]`` amaxes of the sub-row granularity those
    helpers select under tensor parallelism;
  * forward and dgrad round to bf16 once (``bf16(acc * sa * sb + bias)``); the
    reference's dgrad rounds the unscaled product to bf16 first
    (lingua/float8.py:59-77), a work-around for a slow CUTLASS kernel;
  * wgrad is an fp8 product with both operands quantised along the token
    dimension (``config.fp8_wgrad = True``).  Setting it to False restores the
    reference's bf16 ``grad_out.t() @ a`` (lingua/float8.py:123);
  * of the converter's side effects the reset of the dynamo code caches
    (lingua/float8.py:187) is kept -- modules compiled before the swap trace
    afresh afterwards -- while the Inductor flag and the CUDA-graph-tree reset
    (lingua/float8.py:162,189) have no counterpart: no code is generated here;
  * linears applied to the same activation one after the other (w1 / w3, wq /
    wk / wv) share its quantised copy within one forward and one backward
    (``config.share_input_casts``); the reference quantises it once per
    linear.  Same bytes, fewer passes over the activation;
  * the reference's autograd work-around ``b_t + grad_out[:1,:,None]*0``
    (lingua/float8.py:108) is a no-op for finite gradients and is not issued.
"""
import re
import weakref
from dataclasses import dataclass
from typing import Callable, Optional

import torch

from . import ops

# avoid division by zero when calculating scale (same value as the reference)
EPS = 1e-12


@dataclass
class Fp8Config:
    # fp8 wgrad (token-dimension scaling); False = bf16 wgrad as in the reference
    fp8_wgrad: bool = True
    # GEMM tile configuration handed to l8_gemm_nt (0 = library default)
    gemm_algo: int = 0
    # linears that are applied to the very same activation one after the other
    # (w1 / w3 of the MLP, wq / wk / wv of attention) quantise it once per
    # forward and once per backward instead of once each
    share_input_casts: bool = True
    # route Fp8Linear through the torch.library operators of lingua_amd.custom_ops
    # (opaque to torch.compile, nameable in activation-checkpointing policies)
    # instead of the plain autograd.Function
    use_custom_ops: bool = False
    # with fp8_wgrad: quantise the input along the token dimension already in
    # forward and keep that e4m3 [K,M] copy (+ K scales) for wgrad instead of the
    # bf16 input: half the bytes held between forward and backward, the same
    # kernels and the same results (plain autograd.Function route only)
    save_fp8_input: bool = False
    # keep the quantised copies of every weight (row-wise for forward, tensor-wise transposed for dgrad:
    # 2 bytes per parameter) until the weight's version counter moves, so that micro-batches between two
    # optimizer steps (gradient accumulation) and evaluation passes quantise each weight once
    cache_weight_casts: bool = False


config = Fp8Config()


def _col_groups(t: torch.Tensor, amax_t: torch.Tensor) -> int:
    """Number of column groups an amax of shape [R or 1, g] asks for, after checking that the tiling is one
    the kernels serve: whole rows or the whole tensor in the row direction, g equal groups of a multiple of
    16 columns in the other (lingua/float8.py:24-30 divides the operand into amax.shape chunks)."""
    if amax_t.dim() != 2 or amax_t.shape[0] not in (1, t.shape[0]) or amax_t.shape[1] < 1:
        raise RuntimeError(f"scale: unsupported amax shape {tuple(amax_t.shape)} for input {tuple(t.shape)}")
    g = amax_t.shape[1]
    if g > 1 and (t.shape[1] % g or (t.shape[1] // g) % 16):
        raise RuntimeError(f"scale: {t.shape[1]} columns do not split into {g} groups of a multiple of 16")
    return g


def scale(t: torch.Tensor, amax_t: Optional[torch.Tensor] = None):
    """Quantise ``t`` [R,C] bf16: returns ``(t_fp8, scale_t)`` like lingua/float8.py:43-47.

    ``amax_t`` selects the granularity by its shape, as the reference's tile
    broadcast does (lingua/float8.py:24-30): ``[R,1]`` (or None) is row-wise,
    ``[1,1]`` tensor-wise, ``[R,g]`` sub-row-wise -- every row in ``g`` equal
    column groups, each with a scale of its own, which is what the reference
    computes when tensor parallelism shards the reduction dimension over ``g``
    ranks (lingua/float8.py:14-21, :86).
    The values of ``amax_t`` are used as given, as in the reference: a row-wise
    amax whose rows all hold the tensor's amax (what lingua/float8.py:115-118
    builds for dgrad) quantises tensor-wise, and an amax that is not the true
    one (from an earlier step, say) scales by it all the same.  ``None`` asks
    for the fused kernel that finds the row amax in the same pass; only the
    sub-row-wise case always recomputes the group amaxes there.
    """
    if amax_t is None:
        q, s, _ = ops.cast_rowwise(t)
        return q, s
    g = _col_groups(t, amax_t)
    if g > 1:
        if amax_t.shape[0] != t.shape[0]:
            raise RuntimeError(f"scale: unsupported amax shape {tuple(amax_t.shape)} for input {tuple(t.shape)}")
        cs = t.shape[1] // g
        q = torch.empty(t.shape, dtype=torch.float8_e4m3fn, device=t.device)
        s = torch.empty((t.shape[0], g), dtype=torch.float32, device=t.device)
        for j in range(g):
            ops.cast_rowwise(t[:, j * cs:(j + 1) * cs], out_q=q[:, j * cs:(j + 1) * cs], out_scale=s[:, j:j + 1])
        return q, s
    if amax_t.shape[0] == t.shape[0] and t.shape[0] != 1:
        return ops.cast_rowwise_given_amax(t, amax_t)
    return ops.cast_tensorwise(t, amax_t, transpose=False)


def matmul(first, amax_first, second_t, amax_second_t, bias, use_fast_accum: bool = True):
    """lingua/float8.py:50-79: quantise both operands, multiply, scale, add bias.

    ``use_fast_accum`` is accepted for signature parity; accumulation is always
    fp32 on the matrix cores and the scales are always applied in the epilogue.

    With sub-row-wise amaxes (``[R,g]`` and ``[N,g]``) the product is the sum of
    ``g`` partial products, one per column group with that group's scales, each
    rounded to bf16 as the per-rank ``_scaled_mm`` of the reference's
    tensor-parallel case is (lingua/float8.py:65-77 under a Shard(1) placement);
    the partials are then added in fp32 and rounded once, where the reference
    leaves the order of that sum to the all-reduce.
    """
    del use_fast_accum
    q1, s1 = scale(first, amax_first)
    q2, s2 = scale(second_t, amax_second_t)
    g1 = s1.shape[1] if s1.dim() == 2 else 1
    g2 = s2.shape[1] if s2.dim() == 2 else 1
    if g1 == 1 and g2 == 1:
        return ops.gemm_nt(q1, q2, s1, s2, bias, algo=config.gemm_algo)
    if g1 != g2:
        raise RuntimeError(f"matmul: operands are scaled in {g1} and {g2} column groups")
    cs = q1.shape[1] // g1
    acc = None
    for j in range(g1):
        part = ops.gemm_nt(q1[:, j * cs:(j + 1) * cs], q2[:, j * cs:(j + 1) * cs], s1[:, j], s2[:, j],
                           bias if j == 0 else None, algo=config.gemm_algo)
        acc = part.float() if acc is None else acc.add_(part)
    return acc.to(torch.bfloat16)


class _LastCast:
    """Memo of the last activation quantised, one entry per (device, stream): two models that step on two streams
    (or two devices) do not evict each other.  A lookup hits when it sees the same memory (pointer, shape,
    strides, dtype) at the same version counter AND comes from a consumer (weight) that has not used the entry
    yet: the same weight asking again means a new pass over the model, which quantises afresh.  An entry keeps
    its tensor alive, so the address cannot be handed to another tensor while it is cached; a stream's forward
    entry is dropped by the first backward that runs on it and its backward entry by the next forward.  At most
    ``MAX_SLOTS`` streams are remembered (the oldest entry goes first)."""

    MAX_SLOTS = 16

    def __init__(self):
        # slot -> (key, tensor kept alive, value, consumers); tuples are replaced as a whole and dict updates are
        # atomic under the interpreter lock: a reader on another thread (forward and autograd threads both come
        # here) sees either the old entry or the new one
        self.entries = {}

    @staticmethod
    def _slot(t):
        return (t.device.index, torch.cuda.current_stream(t.device).cuda_stream)

    @staticmethod
    def _key(t):
        return (t.data_ptr(), tuple(t.shape), tuple(t.stride()), t.dtype, t.device, t._version,
                torch.cuda.current_stream(t.device).cuda_stream)

    def get(self, t, user):
        # inference tensors have no version counter: nothing would show a write, so they are never shared
        if t.is_inference():
            return None
        entry = self.entries.get(self._slot(t))
        if entry is None or user in entry[3] or entry[0] != self._key(t):
            return None
        entry[3].add(user)
        return entry[2]

    def put(self, t, value, user):
        slot = self._slot(t)
        if t.is_inference():
            self.entries.pop(slot, None)
            return
        self.entries.pop(slot, None)          # re-inserted below: the dict's order is the order of last use
        while len(self.entries) >= self.MAX_SLOTS:
            try:
                self.entries.pop(next(iter(self.entries)), None)
            except (StopIteration, RuntimeError):
                break
        self.entries[slot] = (self._key(t), t, value, {user})

    def clear(self, like=None):
        """Drops the entry of the device and current stream of ``like``, or every entry (``like=None``)."""
        if like is None:
            self.entries.clear()
        elif like.is_cuda:
            self.entries.pop(self._slot(like), None)


_fwd_cast = _LastCast()   # a -> (qa, sa, a_col_amax | None)
_bwd_cast = _LastCast()   # a -> (qat, sat)
_fwd_tcast = _LastCast()  # a -> (qat, sat), made in forward when config.save_fp8_input


class _WeightCasts:
    """Quantised copies of weights, one slot per live weight tensor, valid while pointer, shape, strides, dtype,
    version counter and stream are what they were (an optimizer step advances the version).  A slot holds the
    weight by weak reference only and goes away with it, so the cache never holds more than two bytes per
    parameter of the ``Fp8Linear`` weights that are alive, and a deleted model releases its copies.  Used only
    with ``config.cache_weight_casts``."""

    def __init__(self):
        self.entries = {}   # id(weight) -> {"ref": weakref to the weight, "key": ..., "row": ..., "tw": ...}

    def _slot(self, w):
        if w.is_inference():
            return None
        key = _LastCast._key(w)
        slot = self.entries.get(id(w))
        if slot is not None and slot["ref"]() is not w:
            slot = None             # the id was handed to another object
        if slot is None or slot["key"] != key:
            entries, wid = self.entries, id(w)

            def drop(ref, entries=entries, wid=wid):
                cur = entries.get(wid)
                if cur is not None and cur["ref"] is ref:
                    del entries[wid]

            slot = {"key": key, "ref": weakref.ref(w, drop)}
            self.entries[wid] = slot
        return slot

    def rowwise(self, w):
        slot = self._slot(w) if config.cache_weight_casts else None
        if slot is not None and "row" in slot:
            return slot["row"]
        value = ops.cast_rowwise(w)
        if slot is not None:
            slot["row"] = value
        return value

    def tensorwise_t(self, w, amax_rows):
        slot = self._slot(w) if config.cache_weight_casts else None
        if slot is not None and "tw" in slot:
            return slot["tw"]
        value = ops.cast_tensorwise(w, ops.amax_reduce(amax_rows), transpose=True)
        if slot is not None:
            slot["tw"] = value
        return value

    def clear(self):
        self.entries.clear()


_weight_casts = _WeightCasts()


def weight_cast_rowwise(w):
    """``(q, scale, row amax)`` of a weight, row-wise (the forward operand, lingua/float8.py:87)."""
    return _weight_casts.rowwise(w)


def weight_cast_tensorwise_t(w, amax_rows):
    """``(q [K,N], scale [1,1])`` of a weight [N,K], tensor-wise from its saved row amaxes and written
    transposed (the dgrad operand, lingua/float8.py:111-118)."""
    return _weight_casts.tensorwise_t(w, amax_rows)


def clear_cast_memos() -> None:
    """Forget the shared activation casts.  The memos trust the tensor's version counter, exactly as
    autograd's check of saved tensors does: every PyTorch in-place op and every ``out=`` write of
    ``lingua_amd.ops`` advances it.  A write that bypasses it (``x.data.copy_``, a foreign kernel on
    ``data_ptr()``) between two linears on the same tensor must be followed by this call (or run with
    ``config.share_input_casts = False``)."""
    _fwd_cast.clear()
    _bwd_cast.clear()
    _fwd_tcast.clear()
    _weight_casts.clear()


def set_scale_rule(rule: str) -> None:
    """``"divide"`` (default): scale = clamp(amax) / 448 as a correctly rounded fp32 division -- ATen's CPU kernel, the
    benchmark's statement of the recipe.  ``"times_inverse"``: clamp(amax) * fp32(1/448) -- what ATen's GPU kernel
    makes of ``/ FP8_MAX`` at lingua/float8.py:44 (it multiplies a tensor by the reciprocal of a Python scalar), so
    scales and fp8 bytes equal, bit for bit, those the reference produces on a GPU.  The two differ in the last bit of
    about half of all scales and, because bf16 inputs meet rounding ties of e4m3 exactly, in 0.03-0.1 % of the
    bytes.  Quantised copies kept from before the call are dropped."""
    ops.set_scale_rule(rule)
    clear_cast_memos()


def get_scale_rule() -> str:
    return ops.get_scale_rule()


def linear_forward(a, b_t, bias, need_wgrad_stats: bool, gemm_algo: int):
    """Forward of lingua/float8.py:85-96 on 2-D bf16 operands.  Returns ``(out, amax_b_t, a_col_amax | None)``:
    the two extra tensors are what backward needs beyond ``a`` and ``b_t``."""
    if a.dtype != torch.bfloat16 or b_t.dtype != torch.bfloat16:
        raise RuntimeError(f"Fp8LinearFn: bf16 input and weight required, got {a.dtype} and {b_t.dtype}")
    if not a.is_cuda or a.device != b_t.device:
        raise RuntimeError(f"Fp8LinearFn: input and weight must be on the same GPU, got {a.device} and {b_t.device} "
                           "(there is no CPU path)")
    if a.shape[-1] % 16 or b_t.shape[0] % 16:
        # what torch._scaled_mm tells the reference at lingua/float8.py:65 (both of mat2's dimensions must be
        # divisible by 16); here the forward product could run, but dgrad reduces over out_features
        raise RuntimeError(f"Fp8LinearFn: in_features ({a.shape[-1]}) and out_features ({b_t.shape[0]}) must be multiples of 16")
    # column amaxes of `a` fall out of the row-wise pass; wgrad wants them
    _bwd_cast.clear(a)
    hit = _fwd_cast.get(a, b_t.data_ptr()) if config.share_input_casts else None
    if hit is not None and (hit[2] is not None or not need_wgrad_stats):
        qa, sa, a_col_amax = hit
        if not need_wgrad_stats:
            a_col_amax = None
    else:
        a_col_amax = torch.empty(a.shape[1], dtype=torch.float32, device=a.device) if need_wgrad_stats else None
        qa, sa, _ = ops.cast_rowwise(a, col_amax=a_col_amax)
        if config.share_input_casts:
            _fwd_cast.put(a, (qa, sa, a_col_amax), b_t.data_ptr())
    qb, sb, amax_b_t = weight_cast_rowwise(b_t)
    out = ops.gemm_nt(qa, qb, sa, sb, bias, algo=gemm_algo)
    return out, amax_b_t, a_col_amax


def input_cast_for_wgrad(a, a_col_amax, user):
    """``a`` [M,K] quantised along the token dimension into the [K,M] layout wgrad multiplies with, in forward;
    linears applied to the same activation share one copy."""
    hit = _fwd_tcast.get(a, user) if config.share_input_casts else None
    if hit is not None:
        return hit
    value = ops.cast_colwise_transposed(a, a_col_amax)
    if config.share_input_casts:
        _fwd_tcast.put(a, value, user)
    return value


def linear_backward(grad_out, a, b_t, amax_b_t, a_col_amax, need_a: bool, need_b: bool, need_bias: bool,
                    fp8_wgrad: bool, gemm_algo: int, a_tcast=None):
    """Backward of lingua/float8.py:99-131 (fp8 wgrad optional).  Returns ``(grad_a, grad_b, grad_bias)`` with
    ``None`` where not needed.  ``a_tcast`` = ``(qat [K,M], sat [K,1])`` made in forward stands in for ``a``
    (then ``a`` may be None; fp8 wgrad only)."""
    if grad_out.dtype != torch.bfloat16:
        raise RuntimeError(f"Fp8LinearFn.backward: bf16 grad_out required, got {grad_out.dtype}")
    fp8_wgrad = fp8_wgrad and need_b
    _fwd_cast.clear(grad_out)
    _fwd_tcast.clear(grad_out)
    if a is None and need_b and not (fp8_wgrad and a_tcast is not None):
        raise RuntimeError("Fp8LinearFn.backward: the bf16 input was not saved and no quantised copy stands in for it")

    g_col_amax = None
    if need_a:
        # grad_out row-wise, weight tensor-wise from the row amaxes saved in
        # forward, quantised straight into the [K,N] layout dgrad multiplies with
        g_col_amax = torch.empty(grad_out.shape[1], dtype=torch.float32, device=grad_out.device) if fp8_wgrad else None
        qg, sg, _ = ops.cast_rowwise(grad_out, col_amax=g_col_amax)
        qb, sb = weight_cast_tensorwise_t(b_t, amax_b_t)
        grad_a = ops.gemm_nt(qg, qb, sg, sb, None, algo=gemm_algo)
    else:
        grad_a = None

    if need_b:
        if fp8_wgrad:
            if g_col_amax is None:
                g_col_amax = ops.col_amax(grad_out)
            qgt, sgt = ops.cast_colwise_transposed(grad_out, g_col_amax)
            hit = _bwd_cast.get(a, b_t.data_ptr()) if config.share_input_casts and a_tcast is None else None
            if a_tcast is not None:
                qat, sat = a_tcast
            elif hit is not None:
                qat, sat = hit
            else:
                if a_col_amax is None:
                    a_col_amax = ops.col_amax(a)
                qat, sat = ops.cast_colwise_transposed(a, a_col_amax)
                if config.share_input_casts:
                    _bwd_cast.put(a, (qat, sat), b_t.data_ptr())
            grad_b = ops.gemm_nt(qgt, qat, sgt, sat, None, algo=gemm_algo)
        else:
            grad_b = grad_out.t() @ a
    else:
        grad_b = None

    grad_bias = grad_out.sum(dim=0) if need_bias else None
    return grad_a, grad_b, grad_bias


class Fp8LinearFn(torch.autograd.Function):
    """``out = a @ b_t.T + bias`` with fp8 operands (lingua/float8.py:83-131)."""

    @staticmethod
    def forward(ctx, a, b_t, bias):
        need_wgrad_stats = config.fp8_wgrad and b_t.requires_grad
        out, amax_b_t, a_col_amax = linear_forward(a, b_t, bias, need_wgrad_stats, config.gemm_algo)
        ctx.a_requires_grad = a.requires_grad
        ctx.b_requires_grad = b_t.requires_grad
        ctx.bias_requires_grad = bias.requires_grad if bias is not None else False
        ctx.fp8_wgrad = config.fp8_wgrad
        ctx.gemm_algo = config.gemm_algo
        ctx.kept = "a"
        if need_wgrad_stats and config.save_fp8_input:
            qat, sat = input_cast_for_wgrad(a, a_col_amax, b_t.data_ptr())
            ctx.kept = "a_tcast"
            ctx.save_for_backward(b_t, amax_b_t, qat, sat)
        elif a_col_amax is not None:
            ctx.kept = "a+col"
            ctx.save_for_backward(a, b_t, amax_b_t, a_col_amax)
        else:
            ctx.save_for_backward(a, b_t, amax_b_t)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        a = a_col_amax = a_tcast = None
        if ctx.kept == "a_tcast":
            b_t, amax_b_t, qat, sat = ctx.saved_tensors
            a_tcast = (qat, sat)
        elif ctx.kept == "a+col":
            a, b_t, amax_b_t, a_col_amax = ctx.saved_tensors
        else:
            a, b_t, amax_b_t = ctx.saved_tensors
        return linear_backward(grad_out, a, b_t, amax_b_t, a_col_amax, ctx.a_requires_grad, ctx.b_requires_grad,
                               ctx.bias_requires_grad, ctx.fp8_wgrad, ctx.gemm_algo, a_tcast)


class Fp8Linear(torch.nn.Linear):
    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if config.use_custom_ops:
            from .custom_ops import fp8_linear
            out = fp8_linear(input.flatten(end_dim=-2), self.weight, self.bias)
        else:
            out = Fp8LinearFn.apply(input.flatten(end_dim=-2), self.weight, self.bias)
        out = out.unflatten(0, input.shape[:-1])
        return out


def named_replace(fn: Callable[[torch.nn.Module, str], torch.nn.Module], module: torch.nn.Module, name="") -> torch.nn.Module:
    """Post-order rewrite of a module tree: children first, then the node
    itself; ``fn`` sees dotted names (``""`` for the root)."""
    for child_name, child_module in list(module.named_children()):
        full_name = f"{name}.{child_name}" if name else child_name
        setattr(module, child_name, named_replace(fn, child_module, full_name))
    return fn(module, name)


def convert_linears_to_fp8(root_module: torch.nn.Module, recipe: str, filter: str) -> torch.nn.Module:
    """Swap every exact ``nn.Linear`` whose dotted name matches ``filter`` for an
    ``Fp8Linear`` that shares the same Parameter objects.  Same contract as
    lingua/float8.py:150-191: unknown recipe -> RuntimeError; a matching
    subclass of ``nn.Linear`` (e.g. an already converted layer) -> AssertionError."""
    if recipe not in ["rowwise"]:
        raise RuntimeError(f"Unknown float8 recipe {recipe!r}")

    filter_re = re.compile(filter)

    def replace(module: torch.nn.Module, name: str) -> torch.nn.Module:
        if not isinstance(module, torch.nn.Linear) or not filter_re.search(name):
            return module
        assert type(module) == torch.nn.Linear, str(type(module))
        new_module = Fp8Linear(
            in_features=module.in_features,
            out_features=module.out_features,
            bias=module.bias is not None,
            dtype=module.weight.dtype,
            device=module.weight.device,
        )
        new_module.weight = module.weight
        new_module.bias = module.bias
        return new_module

    out = named_replace(replace, root_module)

    # As lingua/float8.py:187: a model (or a part of it) compiled before the swap holds graphs traced through the
    # old nn.Linear modules; dropping the code caches makes the next call trace the converted modules.  The
    # reference's reset of Inductor's CUDA-graph trees (:189) has no counterpart: nothing here generates code.
    torch._dynamo.reset_code_caches()
    return out
