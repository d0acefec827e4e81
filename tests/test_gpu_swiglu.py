"""GPU parity of the fused SwiGLU kernels and of the fused MLP.

Two stages, so that the floating-point part and the integer part are judged
separately:
  1. the gate itself (h, g1, g3: fp32 exp / division, rounded to bf16) against
     the PyTorch CPU chain of ``oracle.recipe_torch`` -- tolerance: at most two
     bf16 ulps on any element and at least 99.5 % of the elements identical
     (the kernels use the hardware exp2 / reciprocal, about one fp32 ulp each);
     values below 1e-30 in magnitude, where the hardware reciprocal flushes
     subnormal results to zero (silu(-88) = -5e-37), are compared absolutely;
  2. amax, scale, e4m3 bytes and column amaxes against the C oracle applied to
     the kernel's OWN bf16 output -- bit-exact, as for the plain casts.
The fused MLP is compared with the unfused drop-in path (same kernels around a
PyTorch gate) at rel-L2 <= 1e-3 on y and every gradient.
"""
import pytest
import torch

import oracle
from oracle import recipe_torch as rt
from conftest import rel_l2, seeded_bf16
from golden_util import bits_equal

pytestmark = pytest.mark.gpu

ULP_EXACT_FRACTION = 0.995
TINY = 1e-30
MAX_ULPS = 2  # an intermediate that rounds the other way (1 ulp) can move the rounded product by 2
TOL = 1e-3


def bf16_ulp_distance(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """distance in bf16 code steps between two finite bf16 tensors (sign-magnitude -> linear order)"""
    def lin(t):
        u = t.contiguous().view(torch.int16).to(torch.int32) & 0xFFFF
        return torch.where(u >= 0x8000, 0x8000 - u, u)
    return (lin(a) - lin(b)).abs()


def check_close_bf16(got: torch.Tensor, want: torch.Tensor, what: str):
    got, want = got.cpu(), want.cpu()
    finite = torch.isfinite(want.float())
    assert torch.equal(torch.isnan(got.float()), torch.isnan(want.float())), f"{what}: NaN pattern differs"
    tiny = finite & (want.float().abs() < TINY)
    assert float(got[tiny].float().abs().max()) < 2 * TINY if tiny.any() else True, f"{what}: tiny values differ"
    finite = finite & ~tiny
    d = bf16_ulp_distance(got[finite], want[finite])
    assert int(d.max()) <= MAX_ULPS if d.numel() else True, f"{what}: {int(d.max())} bf16 ulps apart"
    exact = float((d == 0).float().mean()) if d.numel() else 1.0
    assert exact >= ULP_EXACT_FRACTION, f"{what}: only {exact:.4%} of the elements identical"


def check_cast_of(x_bf16_gpu, q, s, a=None, col=None, what=""):
    """q / s / amax / col amax must be the C oracle's row-wise cast of x (bit-exact)."""
    x = x_bf16_gpu.cpu()
    qo, so, ao = oracle.cast_rowwise(x)
    assert torch.equal(q.cpu().view(torch.uint8), qo), f"{what}: bytes differ"
    assert bits_equal(s.cpu().reshape(-1), so), f"{what}: scales differ"
    if a is not None:
        assert bits_equal(a.cpu().reshape(-1), ao), f"{what}: amax differ"
    if col is not None:
        assert bits_equal(col.cpu(), oracle.col_amax(x).float()), f"{what}: column amax differ"


SHAPES = [(1, 8), (5, 264), (7, 2048), (300, 1000), (33, 4096), (66, 8192), (21, 11008), (9, 14336), (5, 28672), (3, 32768)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("with_col", [False, True])
def test_forward_gate_and_cast(shape, with_col):
    from lingua_amd import ops
    h1 = seeded_bf16(shape, std=2.0, seed=shape[0] * 17 + shape[1])
    h3 = seeded_bf16(shape, std=1.5, seed=shape[0] * 19 + shape[1] + 1)
    h1[0, 0] = 0.0
    if shape[1] >= 16:
        h1[0, 8:16] = torch.tensor([-100.0, 100.0, -20.0, 20.0, -1e-3, 1e-3, 88.0, -88.0]).to(torch.bfloat16)
    col = torch.zeros(shape[1], dtype=torch.float32, device="cuda") if with_col else None
    h, q, s, a = ops.swiglu_cast_rowwise(h1.cuda(), h3.cuda(), want_h=True, col_amax=col)
    check_close_bf16(h, rt.swiglu_gate(h1, h3), "h")
    check_cast_of(h, q, s, a, col, "forward")
    # without materialising h: same bytes and scales
    col2 = torch.zeros_like(col) if with_col else None
    h_none, q2, s2, a2 = ops.swiglu_cast_rowwise(h1.cuda(), h3.cuda(), want_h=False, col_amax=col2)
    assert h_none is None
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2, s) and torch.equal(a2.view(torch.int16), a.view(torch.int16))
    if with_col:
        assert torch.equal(col2, col)


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("with_col", [False, True])
def test_backward_gate_and_casts(shape, with_col):
    from lingua_amd import ops
    h1 = seeded_bf16(shape, std=2.0, seed=shape[0] * 23 + shape[1])
    h3 = seeded_bf16(shape, std=1.5, seed=shape[0] * 29 + shape[1] + 1)
    dh = seeded_bf16(shape, std=0.01, seed=shape[0] * 31 + shape[1] + 2)
    c1 = torch.zeros(shape[1], dtype=torch.float32, device="cuda") if with_col else None
    c3 = torch.zeros(shape[1], dtype=torch.float32, device="cuda") if with_col else None
    g1, g3, q1, q3, s1, s3 = ops.swiglu_bwd_cast_rowwise(dh.cuda(), h1.cuda(), h3.cuda(), c1, c3)
    w1, w3 = rt.swiglu_gate_bwd(dh, h1, h3)
    check_close_bf16(g1, w1, "g1")
    check_close_bf16(g3, w3, "g3")
    check_cast_of(g1, q1, s1, None, c1, "g1")
    check_cast_of(g3, q3, s3, None, c3, "g3")


def test_strided_inputs_and_nonfinite_rows():
    from lingua_amd import ops
    R, C = 12, 520
    big1 = seeded_bf16((R, C + 24), std=2.0, seed=5).cuda()
    big3 = seeded_bf16((R, C + 40), std=1.0, seed=6).cuda()
    h1, h3 = big1[:, 8:8 + C], big3[:, 16:16 + C]          # row strides differ, 16-byte aligned starts
    h1c, h3c = h1.contiguous(), h3.contiguous()
    h3c[2, 5] = float("inf")
    h3c[4, 7] = float("nan")
    h1c[6, 9] = float("nan")
    big3[2, 16 + 5] = float("inf")
    big3[4, 16 + 7] = float("nan")
    big1[6, 8 + 9] = float("nan")
    a = ops.swiglu_cast_rowwise(h1, h3)
    b = ops.swiglu_cast_rowwise(h1c, h3c)
    for x, y in zip(a, b):
        assert torch.equal(x.view(torch.uint8), y.view(torch.uint8))
    h, q, s, am = a
    hc = h.cpu().float()
    assert torch.isinf(hc[2, 5]) and torch.isnan(hc[4, 7]) and torch.isnan(hc[6, 9])
    # a row with a non-finite amax: scale inf / NaN, bytes NaN codes or zeros exactly as the plain cast does
    q0, s0, a0 = ops.cast_rowwise(h)
    assert torch.equal(q0.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s0.view(torch.int32), s.view(torch.int32))
    assert torch.equal(a0.view(torch.int16), am.view(torch.int16))


@pytest.mark.parametrize("C", [520, 3000, 6000, 11008, 14336])
def test_nonfinite_rows_at_every_kernel_width(C):
    """A row whose amax is infinite or NaN takes the integer conversion in a fix-up loop of its own; one width per
    kernel variant (256 and 512 threads, one to four chunks per thread, and the two-pass kernel), forward with and
    without the bf16 result written out, and backward.  The bytes must equal the plain row-wise cast of the kernel's own
    bf16 output, which the C oracle pins."""
    from lingua_amd import ops
    R = 9
    h1 = seeded_bf16((R, C), std=2.0, seed=C + 1)
    h3 = seeded_bf16((R, C), std=1.5, seed=C + 2)
    dh = seeded_bf16((R, C), std=0.01, seed=C + 3)
    h3[1, 5] = float("inf")
    h3[3, C - 3] = float("nan")
    h1[5, C // 2] = float("nan")
    dh[7, C - 9] = float("inf")
    h1d, h3d, dhd = h1.cuda(), h3.cuda(), dh.cuda()
    h, q, s, am = ops.swiglu_cast_rowwise(h1d, h3d, want_h=True)
    q0, s0, a0 = ops.cast_rowwise(h)
    assert not torch.isfinite(s.cpu().reshape(-1)[[1, 3, 5]]).any() and torch.isfinite(s.cpu().reshape(-1)[[0, 2, 4, 6, 7, 8]]).all()
    assert torch.equal(q0.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s0.view(torch.int32), s.view(torch.int32))
    assert torch.equal(a0.view(torch.int16), am.view(torch.int16))
    _, q2, s2, _ = ops.swiglu_cast_rowwise(h1d, h3d, want_h=False)
    assert torch.equal(q2.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s2.view(torch.int32), s.view(torch.int32))
    g1, g3, q1, q3, s1, s3 = ops.swiglu_bwd_cast_rowwise(dhd, h1d, h3d, None, None)
    for g, qg, sg in ((g1, q1, s1), (g3, q3, s3)):
        q0, s0, _ = ops.cast_rowwise(g)
        assert torch.equal(q0.view(torch.uint8), qg.view(torch.uint8)) and torch.equal(s0.view(torch.int32), sg.view(torch.int32))
    assert not torch.isfinite(s1.cpu().reshape(-1)[[1, 3, 5, 7]]).any()


def test_argument_errors():
    from lingua_amd import ops
    h = seeded_bf16((4, 64)).cuda()
    with pytest.raises(RuntimeError):
        ops.swiglu_cast_rowwise(h, h[:, :32])
    with pytest.raises(RuntimeError):
        ops.swiglu_cast_rowwise(h.float(), h)
    with pytest.raises(RuntimeError):
        ops.swiglu_bwd_cast_rowwise(h, h, h, torch.zeros(64, device="cuda"), None)
    wide = torch.zeros((1, 32768 + 512), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="exceeds"):
        ops.swiglu_bwd_cast_rowwise(wide, wide, wide)


def _mlps(dim, ffn, seed):
    import bench_workloads as callers
    from lingua_amd import convert_linears_to_fp8
    from lingua_amd.swiglu import Fp8FeedForward, fuse_feed_forward
    torch.manual_seed(seed)
    holder = torch.nn.Module()
    holder.feed_forward = callers.FeedForward(dim, ffn).to(device="cuda", dtype=torch.bfloat16)
    plain = convert_linears_to_fp8(holder, "rowwise", r"feed_forward\.")
    fused_holder = torch.nn.Module()
    fused_holder.feed_forward = callers.FeedForward(dim, ffn).to(device="cuda", dtype=torch.bfloat16)
    fused_holder.feed_forward.load_state_dict(holder.feed_forward.state_dict())
    fused = fuse_feed_forward(fused_holder)
    assert isinstance(fused.feed_forward, Fp8FeedForward)
    assert set(fused.feed_forward.state_dict()) == set(plain.feed_forward.state_dict())
    return plain.feed_forward, fused.feed_forward


@pytest.mark.parametrize("wgrad_fp8", [True, False])
@pytest.mark.parametrize("dims", [(256, 768, 96), (1024, 2816, 520)])
def test_fused_mlp_matches_the_unfused_path(dims, wgrad_fp8):
    from lingua_amd import float8
    dim, ffn, tokens = dims
    plain, fused = _mlps(dim, ffn, seed=dim)
    x = seeded_bf16((2, tokens // 2, dim), seed=3).cuda()
    gy = seeded_bf16((2, tokens // 2, dim), std=0.02, seed=4).cuda()
    old = float8.config.fp8_wgrad
    float8.config.fp8_wgrad = wgrad_fp8
    try:
        outs = []
        for mlp in (plain, fused):
            xi = x.clone().requires_grad_(True)
            y = mlp(xi)
            y.backward(gy)
            outs.append((y.detach(), xi.grad, mlp.w1.weight.grad, mlp.w3.weight.grad, mlp.w2.weight.grad))
    finally:
        float8.config.fp8_wgrad = old
    for name, a, b in zip(("y", "dx", "dw1", "dw3", "dw2"), outs[1], outs[0]):
        assert a.shape == b.shape and a.dtype == torch.bfloat16
        assert rel_l2(a, b) <= TOL, (name, rel_l2(a, b))


def test_fused_mlp_partial_requires_grad():
    plain, fused = _mlps(256, 512, seed=9)
    x = seeded_bf16((48, 256), seed=11).cuda()
    gy = seeded_bf16((48, 256), std=0.02, seed=12).cuda()
    # input without gradient (first layer of a network)
    y = fused(x)
    y.backward(gy)
    yp = plain(x)
    yp.backward(gy)
    for n in ("w1", "w2", "w3"):
        assert rel_l2(getattr(fused, n).weight.grad, getattr(plain, n).weight.grad) <= TOL, n
    # frozen w1 / w3: only w2 learns
    for m in (plain, fused):
        for n in ("w1", "w3"):
            getattr(m, n).weight.requires_grad_(False)
        m.zero_grad(set_to_none=True)
        m(x).backward(gy)
    assert fused.w1.weight.grad is None and fused.w3.weight.grad is None
    assert rel_l2(fused.w2.weight.grad, plain.w2.weight.grad) <= TOL


def test_fused_mlp_with_no_tokens():
    plain, fused = _mlps(256, 512, seed=10)
    x = torch.zeros((0, 256), dtype=torch.bfloat16, device="cuda", requires_grad=True)
    y = fused(x)
    assert y.shape == (0, 256)
    y.backward(torch.zeros_like(y))
    assert x.grad.shape == (0, 256)
    for n in ("w1", "w2", "w3"):
        g = getattr(fused, n).weight.grad
        assert g.shape == getattr(fused, n).weight.shape and float(g.float().abs().max()) == 0.0


def test_fuse_feed_forward_rejects_other_modules():
    from lingua_amd.swiglu import fuse_feed_forward
    m = torch.nn.Module()
    m.feed_forward = torch.nn.Sequential(torch.nn.Linear(8, 8))
    with pytest.raises(RuntimeError, match="not a w1/w2/w3"):
        fuse_feed_forward(m)


def test_7b_gate_shapes_properties():
    """[16384, 11008]: row amax of h bounds every dequantised element; q of h equals the plain cast of h."""
    from lingua_amd import ops
    g = torch.Generator(device="cuda").manual_seed(1)
    h1 = (torch.randn((16384, 11008), generator=g, device="cuda") * 1.5).to(torch.bfloat16)
    h3 = torch.randn((16384, 11008), generator=g, device="cuda").to(torch.bfloat16)
    col = torch.zeros(11008, dtype=torch.float32, device="cuda")
    h, q, s, a = ops.swiglu_cast_rowwise(h1, h3, col_amax=col)
    ref = torch.nn.functional.silu(h1) * h3
    d = bf16_ulp_distance(h.cpu(), ref.cpu())
    assert int(d.max()) <= MAX_ULPS and float((d == 0).float().mean()) >= ULP_EXACT_FRACTION
    col0 = torch.zeros_like(col)
    q0, s0, a0 = ops.cast_rowwise(h, col_amax=col0)
    assert torch.equal(q0.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s0, s) and torch.equal(col0, col)
    assert torch.equal(a0.view(torch.int16), a.view(torch.int16))
    dh = (torch.randn((16384, 11008), generator=g, device="cuda") * 0.01).to(torch.bfloat16)
    c1, c3 = torch.zeros_like(col), torch.zeros_like(col)
    g1, g3, q1, q3, s1, s3 = ops.swiglu_bwd_cast_rowwise(dh, h1, h3, c1, c3)
    for gg, qq, ss, cc in ((g1, q1, s1, c1), (g3, q3, s3, c3)):
        cz = torch.zeros_like(col)
        qz, sz, _ = ops.cast_rowwise(gg, col_amax=cz)
        assert torch.equal(qz.view(torch.uint8), qq.view(torch.uint8)) and torch.equal(sz, ss) and torch.equal(cz, cc)
    a1 = h1.detach().clone().requires_grad_(True)
    a3 = h3.detach().clone().requires_grad_(True)
    (torch.nn.functional.silu(a1) * a3).backward(dh)
    for got, want in ((g1, a1.grad), (g3, a3.grad)):
        d = bf16_ulp_distance(got.cpu(), want.cpu())
        assert int(d.max()) <= MAX_ULPS and float((d == 0).float().mean()) >= ULP_EXACT_FRACTION


def test_gate_casts_under_the_gpu_division_rule(gpu_division_rule):
    """The fused gate kernels take their scales from the same helper as the plain casts: under the other division rule
    their bytes and scales follow the oracle under that rule."""
    for shape in [(5, 264), (33, 4096), (21, 11008), (3, 32768)]:
        test_forward_gate_and_cast(shape, True)
        test_backward_gate_and_casts(shape, True)
