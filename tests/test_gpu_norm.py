"""GPU parity of the fused RMSNorm -> row-wise cast kernel and of the Fp8RMSNorm module.

Same two stages as for the fused gate: the floating-point part (y, rstd) against the PyTorch CPU
chain of ``oracle.recipe_torch.rmsnorm`` -- at most one bf16 ulp apart and at least 99.5 % of the
elements identical (only the order of the fp32 sum of squares differs); amax / scale / e4m3 bytes /
column amaxes bit-exact against the C oracle applied to the kernel's own bf16 output.
"""
import pytest
import torch

import oracle
from oracle import recipe_torch as rt
from conftest import rel_l2, seeded_bf16
from golden_util import bits_equal
from test_gpu_swiglu import bf16_ulp_distance, check_cast_of

pytestmark = pytest.mark.gpu

EPS = 1e-5


def check_y(y, want):
    d = bf16_ulp_distance(y.cpu(), want.cpu())
    assert int(d.max()) <= 1, f"{int(d.max())} bf16 ulps apart"
    assert float((d == 0).float().mean()) >= 0.995


@pytest.mark.parametrize("shape", [(1, 8), (5, 264), (300, 1000), (33, 2048), (17, 4096), (9, 8192)])
@pytest.mark.parametrize("w_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("with_col", [False, True])
def test_norm_and_cast(shape, w_dtype, with_col):
    from lingua_amd import ops
    x = seeded_bf16(shape, std=3.0, seed=shape[0] * 37 + shape[1])
    x[0, 0] = 0.0
    w = (1.0 + 0.1 * torch.randn(shape[1], generator=torch.Generator().manual_seed(shape[1]))).to(w_dtype)
    col = torch.zeros(shape[1], dtype=torch.float32, device="cuda") if with_col else None
    y, q, s, rstd = ops.rmsnorm_cast_rowwise(x.cuda(), w.cuda(), EPS, col_amax=col)
    check_y(y, rt.rmsnorm(x, w, EPS))
    xf = x.float()
    want_rstd = torch.rsqrt((xf * xf).mean(-1, keepdim=True) + EPS)
    assert torch.allclose(rstd.cpu(), want_rstd, rtol=2e-6, atol=0)
    check_cast_of(y, q, s, None, col, "norm")
    # without the cast: same y
    y2, q2, s2, r2 = ops.rmsnorm_cast_rowwise(x.cuda(), w.cuda(), EPS, want_q=False, want_rstd=False)
    assert q2 is None and s2 is None and r2 is None and torch.equal(y2.view(torch.int16), y.view(torch.int16))


@pytest.mark.parametrize("shape", [(1, 8), (5, 264), (300, 1000), (1027, 2048), (17, 4096), (9, 8192)])
@pytest.mark.parametrize("w_dtype", [torch.bfloat16, torch.float32])
def test_norm_backward(shape, w_dtype):
    """gx, gw of the fused backward against autograd through the oracle's eager chain (fp32 sums in another
    order: rel-L2 <= 1e-3 on the bf16 gx, 1e-4 on the fp32 gw); gw is reproducible bit for bit run to run."""
    from lingua_amd import ops
    x = seeded_bf16(shape, std=3.0, seed=shape[0] * 41 + shape[1])
    gy = seeded_bf16(shape, std=0.05, seed=shape[0] * 43 + shape[1] + 1)
    w = (1.0 + 0.1 * torch.randn(shape[1], generator=torch.Generator().manual_seed(shape[1]))).to(w_dtype)
    xa = x.clone().requires_grad_(True)
    wa = w.clone().requires_grad_(True)
    rt.rmsnorm(xa, wa, EPS).backward(gy)
    _, _, _, rstd = ops.rmsnorm_cast_rowwise(x.cuda(), w.cuda(), EPS, want_q=False)
    gx, gw = ops.rmsnorm_bwd(gy.cuda(), x.cuda(), w.cuda(), rstd)
    assert gx.dtype == torch.bfloat16 and gw.dtype == torch.float32
    assert rel_l2(gx, xa.grad) <= 1e-3
    assert rel_l2(gw, wa.grad.float()) <= (1e-4 if w_dtype == torch.float32 else 5e-3)   # bf16 weight: autograd rounds gw to bf16
    gx2, gw2 = ops.rmsnorm_bwd(gy.cuda(), x.cuda(), w.cuda(), rstd)
    assert torch.equal(gw2, gw) and torch.equal(gx2.view(torch.int16), gx.view(torch.int16))


def test_zero_rows_and_nonfinite():
    from lingua_amd import ops
    x = seeded_bf16((6, 512), seed=2)
    x[1] = 0.0                      # rstd = 1/sqrt(eps), y = 0, scale floor
    x[3, 7] = float("nan")
    x[4, 9] = float("inf")
    w = torch.ones(512, dtype=torch.bfloat16)
    y, q, s, rstd = ops.rmsnorm_cast_rowwise(x.cuda(), w.cuda(), EPS)
    want = rt.rmsnorm(x, w, EPS)
    yc = y.cpu()
    assert torch.equal(torch.isnan(yc.float()), torch.isnan(want.float()))
    assert float(yc[1].float().abs().max()) == 0.0 and s.cpu().view(torch.int32)[1].item() == 0x2720D7C5
    assert abs(float(rstd[1]) * (EPS ** 0.5) - 1.0) < 1e-6
    q0, s0, _ = ops.cast_rowwise(y)
    assert torch.equal(q0.view(torch.uint8), q.view(torch.uint8)) and torch.equal(s0.view(torch.int32), s.view(torch.int32))


def test_argument_errors():
    from lingua_amd import ops
    x = seeded_bf16((4, 64)).cuda()
    with pytest.raises(RuntimeError):
        ops.rmsnorm_cast_rowwise(x, torch.ones(32, device="cuda"), EPS)
    with pytest.raises(RuntimeError):
        ops.rmsnorm_cast_rowwise(x.float(), torch.ones(64, device="cuda"), EPS)
    wide = torch.zeros((1, 8192 + 512), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="exceeds"):
        ops.rmsnorm_cast_rowwise(wide, torch.ones(8192 + 512, device="cuda"), EPS)


class _Block(torch.nn.Module):
    """norm -> three linears on the same normalised activation, as an attention block does"""

    def __init__(self, dim):
        super().__init__()
        from bench_workloads import RMSNorm
        self.attention_norm = RMSNorm(dim, EPS)
        self.wq = torch.nn.Linear(dim, dim, bias=False)
        self.wk = torch.nn.Linear(dim, dim // 2, bias=False)
        self.wv = torch.nn.Linear(dim, dim // 2, bias=False)

    def forward(self, x):
        h = self.attention_norm(x)
        return self.wq(h), self.wk(h), self.wv(h)


def test_module_feeds_the_linears_without_a_cast_of_their_own():
    from lingua_amd import convert_linears_to_fp8, ops
    from lingua_amd.norm import Fp8RMSNorm, fuse_rmsnorm
    torch.manual_seed(4)
    plain = convert_linears_to_fp8(_Block(512).to(device="cuda", dtype=torch.bfloat16), "rowwise", r"w[qkv]$")
    fused = convert_linears_to_fp8(_Block(512).to(device="cuda", dtype=torch.bfloat16), "rowwise", r"w[qkv]$")
    fused.load_state_dict(plain.state_dict())
    with torch.no_grad():
        for m in (plain, fused):
            m.attention_norm.weight.add_(0.1 * torch.randn_like(m.attention_norm.weight))
        fused.attention_norm.weight.copy_(plain.attention_norm.weight)
    fused = fuse_rmsnorm(fused)
    assert isinstance(fused.attention_norm, Fp8RMSNorm)
    assert fused.attention_norm.weight.data_ptr() != plain.attention_norm.weight.data_ptr()
    assert set(fused.state_dict()) == set(plain.state_dict())
    x = seeded_bf16((2, 48, 512), std=2.0, seed=8).cuda()
    gs = [seeded_bf16((2, 48, n), std=0.02, seed=9 + i).cuda() for i, n in enumerate((512, 256, 256))]

    def run(m):
        rec = []
        ops.kernel_timer = rec
        try:
            xi = x.clone().requires_grad_(True)
            outs = m(xi)
            n_casts = sum(1 for r in rec if r[0] == "cast_rowwise")
            torch.autograd.backward(outs, gs)
        finally:
            ops.kernel_timer = None
        grads = [xi.grad, m.attention_norm.weight.grad, m.wq.weight.grad, m.wk.weight.grad, m.wv.weight.grad]
        return [o.detach() for o in outs] + grads, n_casts

    got, casts_fused = run(fused)
    want, casts_plain = run(plain)
    assert casts_plain == 4 and casts_fused == 3      # activation once + three weights vs. weights only
    for name, a, b in zip(("q", "k", "v", "dx", "dnorm_w", "dwq", "dwk", "dwv"), got, want):
        assert rel_l2(a, b) <= 2e-3, (name, rel_l2(a, b))


def test_fuse_rmsnorm_rejects_other_modules():
    from lingua_amd.norm import fuse_rmsnorm
    m = torch.nn.Module()
    m.ffn_norm = torch.nn.LayerNorm(8)
    with pytest.raises(RuntimeError, match="not an RMSNorm"):
        fuse_rmsnorm(m)


def test_small_llama_with_fused_gate_and_norms_matches_the_drop_in_model():
    """A 3-layer Llama in bf16, through convert_linears_to_fp8 alone, and with fuse_feed_forward + fuse_rmsnorm
    on top.  Every last-bit difference in an activation re-rolls the e4m3 rounding downstream, so the two fp8
    models are not compared with each other directly: each gradient of the fused model must be as close to the
    bf16 model's as the drop-in model's is (within a quarter more), and the losses must agree."""
    from lingua_amd import convert_linears_to_fp8
    from bench_workloads import Llama
    from lingua_amd.norm import Fp8RMSNorm, fuse_rmsnorm
    from lingua_amd.swiglu import Fp8FeedForward, fuse_feed_forward
    cfg = dict(n_layers=3, dim=512, n_heads=4, ffn_dim=1536, vocab=1000)
    models = []
    for kind in ("bf16", "fp8", "fp8-fused"):
        with torch.device("cuda"):
            m = Llama(**cfg).to(torch.bfloat16)
        m.init_weights(0.05, seed=1)
        with torch.no_grad():
            for name, p in m.named_parameters():
                if name.endswith("norm.weight"):
                    p.add_(0.1 * torch.randn(p.shape, generator=torch.Generator().manual_seed(len(name))).to(p.device, p.dtype))
        if kind != "bf16":
            m = convert_linears_to_fp8(m, "rowwise", r"layers\.[0-9]+\.")
        if kind == "fp8-fused":
            keys = list(m.state_dict().keys())
            m = fuse_rmsnorm(fuse_feed_forward(m))
            assert list(m.state_dict().keys()) == keys
            assert sum(isinstance(x, Fp8RMSNorm) for x in m.modules()) == 6
            assert sum(isinstance(x, Fp8FeedForward) for x in m.modules()) == 3
            assert not isinstance(m.norm, Fp8RMSNorm)
        models.append(m)
    g = torch.Generator().manual_seed(2)
    tokens = torch.randint(0, cfg["vocab"], (2, 256), generator=g).cuda()
    labels = torch.randint(0, cfg["vocab"], (2, 256), generator=g).cuda()
    losses = []
    for m in models:
        loss = m(tokens, labels)
        loss.backward()
        losses.append(float(loss.detach()))
    assert abs(losses[1] - losses[2]) <= 2e-3 * abs(losses[1]), losses
    assert abs(losses[0] - losses[2]) <= 2e-2 * abs(losses[0]), losses
    ref, plain, fused = (dict(m.named_parameters()) for m in models)
    for n in ref:
        e_plain, e_fused = rel_l2(plain[n].grad, ref[n].grad), rel_l2(fused[n].grad, ref[n].grad)
        assert e_fused <= 1.25 * e_plain + 1e-3, (n, e_plain, e_fused)


def test_fused_feed_forward_takes_the_norm_output_already_quantised():
    """ffn_norm -> feed_forward with both fused: the norm files its output quantised (with column amaxes in
    training), and the fused SwiGLU takes that copy instead of casting the activation again -- one row-wise cast
    fewer per block, identical results (the same kernel arithmetic produced the copy either way)."""
    from lingua_amd import float8, ops
    from lingua_amd.norm import Fp8RMSNorm
    from lingua_amd.swiglu import Fp8FeedForward
    from bench_workloads import FeedForward
    torch.manual_seed(4)
    ff = FeedForward(512, 1024).to(device="cuda", dtype=torch.bfloat16)
    norm = Fp8RMSNorm(512, 1e-5).to(device="cuda", dtype=torch.bfloat16)
    fused = Fp8FeedForward(ff.w1, ff.w3, ff.w2)
    x = seeded_bf16((3, 40, 512), std=1.5, seed=19).cuda()
    g = seeded_bf16((3, 40, 512), std=0.02, seed=20).cuda()

    def run(share):
        old = float8.config.share_input_casts
        float8.config.share_input_casts = share
        rec = []
        ops.kernel_timer = rec
        try:
            for p in list(ff.parameters()) + [norm.weight]:
                p.grad = None
            xi = x.clone().requires_grad_(True)
            y = fused(norm(xi))
            n_fwd = sum(1 for r in rec if r[0] == "cast_rowwise")
            y.backward(g)
        finally:
            ops.kernel_timer = None
            float8.config.share_input_casts = old
        return [y.detach(), xi.grad] + [p.grad.clone() for p in ff.parameters()], n_fwd

    got, n_shared = run(True)
    want, n_apart = run(False)
    assert n_apart == 4 and n_shared == 3          # x + three weights against the three weights only
    for a, b in zip(got, want):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_norm_cast_under_the_gpu_division_rule(gpu_division_rule):
    for shape in [(5, 264), (300, 1000), (17, 4096), (9, 8192)]:
        test_norm_and_cast(shape, torch.bfloat16, True)
