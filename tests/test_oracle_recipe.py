"""Pins the oracle's recipe-level functions (CPU only): the C restatement
against the PyTorch-op restatement, both against the committed golden
vectors, and the product against exact integer arithmetic and an fp64 loop."""
import pytest
import torch

import oracle
from oracle import recipe_torch as rt
from conftest import rel_l2, seeded_bf16
from golden_util import bits_equal, fp8_equal_mod_nan_sign, load_golden


def test_golden_quantisation_both_oracles():
    g = load_golden()
    x, w, go = g["x"], g["w"], g["go"]
    for name, t in (("x", x), ("w", w), ("g", go)):
        q, s, a = oracle.cast_rowwise(t)
        assert torch.equal(q, g["q_" + name]), name
        assert bits_equal(s, g["s_" + name]), name
        qt, st = rt.scale(t, rt.row_amax(t))
        assert torch.equal(qt.view(torch.uint8), g["q_" + name])
        assert bits_equal(st.reshape(-1), g["s_" + name])
    assert bits_equal(oracle.row_amax(x), g["amax_x"])
    # dgrad weight: tensor-wise from row amaxes, transposed layout
    qwt, swt = oracle.cast_tensorwise(w, oracle.amax_of_amaxes(oracle.row_amax(w)), transpose=True)
    assert torch.equal(qwt, g["q_wt"])
    assert bits_equal(swt.expand(g["s_wt"].shape).contiguous(), g["s_wt"])
    # wgrad operands
    for name, t in (("gt", go), ("xt", x)):
        q, s = oracle.cast_colwise_transposed(t)
        assert torch.equal(q, g["q_" + name]), name
        assert bits_equal(s, g["s_" + name]), name
    q, s = oracle.cast_tensorwise(x)
    assert torch.equal(q, g["q_x_tw"]) and bits_equal(s, g["s_x_tw"])


def test_golden_edge_rows():
    g = load_golden()
    q, s = g["q_x"], g["s_x"]
    assert (q[3] == 0x00).all() and (q[4] == 0x80).all() and (q[5] == 0x00).all()
    for r in (3, 4, 5):
        assert s[r].view(torch.int32).item() == 0x2720D7C5
    assert q[6, 0] == 0x7E and q[6, 1] == 0x00
    # row 7 has amax 448 -> scale exactly 1 -> codes are the RNE of the integers
    assert s[7].item() == 1.0
    want = g["x"][7].float().to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(q[7], want)
    assert q[7, 17] == 0x58 and q[7, 19] == 0x5A  # 17 -> 16, 19 -> 20
    # every row with a non-zero amax holds the code of +-448
    nz = g["amax_x"].float() >= 1e-12
    assert ((q[nz] & 0x7F).amax(dim=1) == 0x7E).all()


def test_golden_products_both_oracles():
    g = load_golden()
    x, w, go, bias = g["x_prod"], g["w"], g["go"], g["bias"]
    for got, want in ((oracle.linear_forward(x, w, bias), g["y"]),
                      (oracle.linear_dgrad(go, w), g["dx"]),
                      (oracle.linear_wgrad_fp8(go, x), g["dw_fp8"])):
        fin = want.float().isfinite()
        assert torch.equal(fin, got.float().isfinite())
        assert rel_l2(got.float()[fin], want.float()[fin]) <= 1e-3
    # the bf16 wgrad of the reference and the fp8 wgrad agree to quantisation noise
    a = g["dw_fp8"].float()
    b = g["dw_bf16"].float()
    ok = b.isfinite() & a.isfinite()
    assert rel_l2(a[ok], b[ok]) < 0.1


@pytest.mark.parametrize("shape", [(1, 8), (5, 16), (33, 520), (64, 1000)])
def test_c_oracle_equals_torch_chain(shape):
    x = seeded_bf16(shape, seed=11)
    x[0, 0] = 0
    q, s, a = oracle.cast_rowwise(x)
    qt, st = rt.scale(x, rt.row_amax(x))
    assert torch.equal(q, qt.view(torch.uint8)) and bits_equal(s, st.reshape(-1))
    q2, s2 = oracle.cast_colwise_transposed(x)
    xt = x.t().contiguous()
    q2t, s2t = rt.scale(xt, rt.row_amax(xt))
    assert torch.equal(q2, q2t.view(torch.uint8)) and bits_equal(s2, s2t.reshape(-1))
    # transposed == row-wise of the transpose, and amax handed in == amax computed
    q3, s3, _ = oracle.cast_rowwise(xt)
    assert torch.equal(q2, q3) and bits_equal(s2, s3)
    q4, s4 = oracle.cast_colwise_transposed(x, oracle.col_amax(x))
    assert torch.equal(q2, q4) and bits_equal(s2, s4)
    # tensor-wise: transpose flag only permutes
    qa, sa = oracle.cast_tensorwise(x)
    qb, sb = oracle.cast_tensorwise(x, transpose=True)
    assert torch.equal(qa.t().contiguous(), qb) and bits_equal(sa, sb)
    qc, sc = rt.scale(x, x.abs().amax().reshape(1, 1))
    assert torch.equal(qa, qc.view(torch.uint8)) and bits_equal(sa, sc.reshape(-1))


def test_nonfinite_rows():
    x = seeded_bf16((4, 32), seed=5)
    x[1, 3] = float("inf")
    x[2, 5] = float("nan")
    q, s, a = oracle.cast_rowwise(x)
    qt, st = rt.scale(x, rt.row_amax(x))
    assert fp8_equal_mod_nan_sign(q, qt)
    assert s[1].isinf() and s[2].isnan()
    # inf row: the inf element is NaN (inf * 0), every finite element is +-0
    assert (q[1, 3] & 0x7F) == 0x7F
    rest = torch.cat([q[1, :3], q[1, 4:]])
    assert ((rest & 0x7F) == 0).all()
    assert ((q[2] & 0x7F) == 0x7F).all()


def test_gemm_exact_small_integers():
    # operands in {-1,0,1}: every partial sum is an integer of magnitude <= K <= 256, exact in fp32 and in bf16,
    # so the result must equal the integer matmul bit for bit whatever the accumulation order
    g = torch.Generator().manual_seed(7)
    M, N, K = 19, 23, 96
    A = torch.randint(-1, 2, (M, K), generator=g).float()
    B = torch.randint(-1, 2, (N, K), generator=g).float()
    qa, qb = A.to(torch.float8_e4m3fn), B.to(torch.float8_e4m3fn)
    assert torch.equal(qa.float(), A)
    got = oracle.gemm_nt(qa.view(torch.uint8), qb.view(torch.uint8), torch.tensor([0.5]), torch.tensor([4.0]))
    want = (A.long() @ B.long().t()) * 2
    assert torch.equal(got.double(), want.double())
    # per-row power-of-two scales stay exact too
    sa = torch.tensor([2.0 ** (i % 5 - 2) for i in range(M)])
    sb = torch.tensor([2.0 ** (i % 3) for i in range(N)])
    got = oracle.gemm_nt(qa.view(torch.uint8), qb.view(torch.uint8), sa, sb)
    want = (A.long() @ B.long().t()).double() * sa.double()[:, None] * sb.double()[None, :]
    assert torch.equal(got.double(), want)


def test_gemm_vs_f64_triple_loop_and_torch():
    g = torch.Generator().manual_seed(8)
    M, N, K = 17, 29, 80
    qa = torch.randint(0, 256, (M, K), generator=g, dtype=torch.int32).to(torch.uint8)
    qb = torch.randint(0, 256, (N, K), generator=g, dtype=torch.int32).to(torch.uint8)
    qa[(qa & 0x7F) == 0x7F] = 0x3C
    qb[(qb & 0x7F) == 0x7F] = 0x3C
    sa = torch.rand(M, generator=g) + 0.5
    sb = torch.rand(N, generator=g) + 0.5
    bias = torch.randn(N, generator=g).to(torch.bfloat16)
    ref64 = oracle.gemm_nt(qa, qb, sa, sb, bias, f64=True)
    # independent: torch fp64 matmul of torch-decoded operands
    A = qa.view(torch.float8_e4m3fn).double() * sa.double()[:, None]
    B = qb.view(torch.float8_e4m3fn).double() * sb.double()[:, None]
    want = A @ B.t() + bias.double()
    assert torch.allclose(ref64, want, rtol=1e-12, atol=1e-9)
    got = oracle.gemm_nt(qa, qb, sa, sb, bias)
    assert rel_l2(got, want.to(torch.bfloat16)) < 2e-3
    assert rel_l2(got.double(), want) < 4e-3  # bf16 rounding alone is ~1.7e-3
    # scalar scale modes
    got_s = oracle.gemm_nt(qa, qb, sa[:1], sb[:1])
    want_s = (qa.view(torch.float8_e4m3fn).double() @ qb.view(torch.float8_e4m3fn).double().t()) * sa[0].double() * sb[0].double()
    assert rel_l2(got_s.double(), want_s) < 4e-3


def test_linear_products_c_vs_torch_chain():
    x = seeded_bf16((96, 256), seed=21)
    w = seeded_bf16((72, 256), std=0.02, seed=22)
    go = seeded_bf16((96, 72), std=1e-2, seed=23)
    assert rel_l2(oracle.linear_forward(x, w), rt.linear_forward(x, w)) < 1e-3
    assert rel_l2(oracle.linear_dgrad(go, w), rt.linear_dgrad(go, w)) < 1e-3
    assert rel_l2(oracle.linear_wgrad_fp8(go, x), rt.linear_wgrad_fp8(go, x)) < 1e-3
    # fp8 products track the bf16 products to quantisation noise
    assert rel_l2(rt.linear_forward(x, w), (x.float() @ w.float().t())) < 0.06
    assert rel_l2(rt.linear_wgrad_fp8(go, x), rt.linear_wgrad_bf16(go, x)) < 0.06


def test_col_sum():
    go = seeded_bf16((50, 24), seed=31)
    assert rel_l2(oracle.col_sum(go), go.float().sum(0)) < 5e-3


def test_swiglu_gate_oracle_against_float64_closed_forms():
    """oracle.recipe_torch.swiglu_gate / swiglu_gate_bwd are the reference's own eager ops; pin them
    against the closed forms in float64: silu(x) = x / (1 + e^-x), d silu = s (1 + x (1 - s))."""
    g = torch.Generator().manual_seed(77)
    h1 = (torch.randn((64, 256), generator=g) * 3).to(torch.bfloat16)
    h3 = (torch.randn((64, 256), generator=g) * 2).to(torch.bfloat16)
    dh = (torch.randn((64, 256), generator=g) * 0.1).to(torch.bfloat16)
    h = rt.swiglu_gate(h1, h3)
    x, y, d = h1.double(), h3.double(), dh.double()
    sig = 1.0 / (1.0 + torch.exp(-x))
    want_h = x * sig * y
    # two bf16 roundings (silu, product): each at most half an ulp = 2^-8 relative
    assert h.dtype == torch.bfloat16
    assert float(((h.double() - want_h).abs() / want_h.abs().clamp_min(1e-30)).max()) <= 2.0 ** -6.95
    g1, g3 = rt.swiglu_gate_bwd(dh, h1, h3)
    want_g3 = d * (x * sig)
    want_g1 = d * y * sig * (1 + x * (1 - sig))
    assert float(((g3.double() - want_g3).abs() / want_g3.abs().clamp_min(1e-30)).max()) <= 2.0 ** -6.95
    # the factor 1 + x (1 - s) cancels near x = -1.278: absolute bound scaled by |d y|
    assert float(((g1.double() - want_g1).abs() / (d * y).abs().clamp_min(1e-30)).max()) <= 1.1 * 2.0 ** -6.95
    # known answers: silu(0) = 0, silu'(0) = 1/2, silu(40) = 40, silu(-40) = -40 e^-40
    z = torch.tensor([[0.0, 40.0, -40.0]], dtype=torch.bfloat16)
    one = torch.ones_like(z)
    hz = rt.swiglu_gate(z, one).double()[0].tolist()
    assert hz[0] == 0.0 and hz[1] == 40.0 and abs(hz[2] / (-40.0 * 4.248354255291589e-18) - 1.0) <= 2.0 ** -7.9
    g1z, g3z = rt.swiglu_gate_bwd(one, z, one)
    assert g1z[0, :2].tolist() == [0.5, 1.0] and abs(float(g1z[0, 2])) < 1e-14
    assert g3z[0, :2].tolist() == [0.0, 40.0]


def test_rmsnorm_oracle_against_float64():
    """oracle.recipe_torch.rmsnorm is the reference's eager op chain; pin it against x / sqrt(mean(x^2) + eps) * w
    in float64 (one bf16 rounding at the end: half an ulp = 2^-8 relative, plus fp32 noise)."""
    g = torch.Generator().manual_seed(78)
    x = (torch.randn((48, 320), generator=g) * 4).to(torch.bfloat16)
    w = (1 + 0.2 * torch.randn(320, generator=g)).to(torch.bfloat16)
    y = rt.rmsnorm(x, w, 1e-5)
    xd = x.double()
    want = xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + 1e-5) * w.double()
    assert y.dtype == torch.bfloat16
    assert float(((y.double() - want).abs() / want.abs().clamp_min(1e-30)).max()) <= 2.0 ** -7.99
    # a constant row c normalises to sign(c) * w (for |c| >> sqrt(eps)); a zero row stays zero
    z = torch.full((1, 64), -3.0, dtype=torch.bfloat16)
    assert torch.equal(rt.rmsnorm(z, torch.ones(64, dtype=torch.bfloat16), 1e-6), torch.full((1, 64), -1.0, dtype=torch.bfloat16))
    assert float(rt.rmsnorm(torch.zeros((1, 64), dtype=torch.bfloat16), torch.ones(64), 1e-6).abs().max()) == 0.0


def test_tiled_scale_oracle_against_slices_and_a_plain_loop():
    """The [R,g] branch of the oracle's scale(): (1) every column group must come out as the row-wise C oracle
    (pinned by the golden vectors) quantises that group on its own; (2) the tile expansion is checked element by
    element against index arithmetic on a shape where a transposed or row/column-swapped expansion differs;
    (3) g = 1 and [1,1] reduce to the branches the golden vectors cover."""
    x = seeded_bf16((6, 96), std=2.0, seed=31)
    x[2, 32:64] = 0.0
    x[4, 5] = 300.0
    for g in (1, 2, 3, 6):
        amax = rt.subrow_amax(x, g)
        assert amax.shape == (6, g) and amax.dtype == torch.bfloat16
        q, s = rt.scale(x, amax)
        cs = 96 // g
        for j in range(g):
            qj, sj, aj = oracle.cast_rowwise(x[:, j * cs:(j + 1) * cs].contiguous())
            assert torch.equal(q[:, j * cs:(j + 1) * cs].view(torch.uint8), qj), (g, j)
            assert bits_equal(s[:, j].contiguous(), sj) and bits_equal(amax[:, j].contiguous(), aj)
    b = torch.arange(6, dtype=torch.float32).reshape(2, 3)
    e = rt.tile_broadcast(b, (4, 12))
    for r in range(4):
        for c in range(12):
            assert e[r, c] == b[r // 2, c // 4]
    q1, s1 = rt.scale(x, x.abs().amax().reshape(1, 1))
    q2, s2 = oracle.cast_tensorwise(x)
    assert torch.equal(q1.view(torch.uint8), q2) and bits_equal(s1.reshape(-1), s2.reshape(-1))


def test_subrow_product_oracle_reduces_to_known_cases():
    """dequant_matmul with g scale columns: equal to the plain product when all groups share one scale and the
    values are small integers (every partial and the sum are exact in bf16), and group j's scales must reach
    group j's columns only (a product with one group zeroed loses exactly that group's term)."""
    g, cs = 4, 16
    gen = torch.Generator().manual_seed(5)
    qa = torch.randint(-2, 3, (5, g * cs), generator=gen).float().to(torch.float8_e4m3fn)
    qb = torch.randint(-2, 3, (7, g * cs), generator=gen).float().to(torch.float8_e4m3fn)
    ones_a, ones_b = torch.ones(5, g), torch.ones(7, g)
    want = (qa.float() @ qb.float().t())
    assert torch.equal(rt.dequant_matmul(qa, ones_a, qb, ones_b).float(), want)
    sa = torch.tensor([1.0, 2.0, 4.0, 8.0]).repeat(5, 1)
    sb = torch.tensor([1.0, 0.5, 0.25, 0.125]).repeat(7, 1)
    assert torch.equal(rt.dequant_matmul(qa, sa, qb, sb).float(), want)      # sa*sb == 1 in every group
    sa0 = ones_a.clone()
    sa0[:, 2] = 0.0
    lost = qa[:, 2 * cs:3 * cs].float() @ qb[:, 2 * cs:3 * cs].float().t()
    assert torch.equal(rt.dequant_matmul(qa, sa0, qb, ones_b).float(), want - lost)


@pytest.mark.parametrize("shape", [(5, 16), (33, 520), (64, 1000)])
def test_c_oracle_equals_torch_chain_under_the_gpu_division_rule(shape):
    """Both restatements under oracle.scale_rule("times_inverse"): same bytes and scales as each other in every
    layout, and not the same as under the default rule (bf16 inputs meet e4m3's rounding ties exactly, so the last bit
    of a scale decides bytes)."""
    x = seeded_bf16(shape, seed=11)
    x[0, 0] = 0
    q0, s0, _ = oracle.cast_rowwise(x)
    with oracle.scale_rule("times_inverse"):
        q, s, a = oracle.cast_rowwise(x)
        qt, st = rt.scale(x, rt.row_amax(x))
        assert torch.equal(q, qt.view(torch.uint8)) and bits_equal(s, st.reshape(-1))
        q2, s2 = oracle.cast_colwise_transposed(x)
        xt = x.t().contiguous()
        q2t, s2t = rt.scale(xt, rt.row_amax(xt))
        assert torch.equal(q2, q2t.view(torch.uint8)) and bits_equal(s2, s2t.reshape(-1))
        qa, sa = oracle.cast_tensorwise(x)
        qc, sc = rt.scale(x, x.abs().amax().reshape(1, 1))
        assert torch.equal(qa, qc.view(torch.uint8)) and bits_equal(sa, sc.reshape(-1))
    assert not bits_equal(s, s0)
    q1, s1, _ = oracle.cast_rowwise(x)          # the rule is back to the default outside the block
    assert torch.equal(q1, q0) and bits_equal(s1, s0)
