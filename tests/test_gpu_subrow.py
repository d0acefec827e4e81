"""GPU parity of sub-row-wise scaling: amax of shape [R,g], the granularity the reference uses when tensor
parallelism shards the reduction dimension over g ranks (lingua/float8.py:14-21, :24-30, :86).  On one GPU
scale() and matmul() serve it group by group on the row-wise kernels; e4m3 bytes and scales are bit-exact
against the oracle, the product within rel-L2 1e-3 of the oracle's sum of bf16 partial products."""
import pytest
import torch

import oracle
from oracle import recipe_torch as rt
from conftest import rel_l2, seeded_bf16
from golden_util import bits_equal

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,g", [((6, 96), 2), ((6, 96), 3), ((1, 64), 4), ((300, 1024), 8), ((65, 4096), 2)])
def test_scale_with_column_groups(shape, g):
    from lingua_amd import float8 as f8
    x = seeded_bf16(shape, std=2.0, seed=shape[0] + g)
    x[0, : shape[1] // g] = 0.0                    # one all-zero group: scale floor in that group only
    x[-1, shape[1] - 1] = 200.0                    # an outlier confined to the last group
    amax = rt.subrow_amax(x, g)
    q, s = f8.scale(x.cuda(), amax.cuda())
    want_q, want_s = rt.scale(x, amax)
    assert q.shape == x.shape and s.shape == (shape[0], g) and s.dtype == torch.float32
    assert torch.equal(q.cpu().view(torch.uint8), want_q.view(torch.uint8))
    assert bits_equal(s.cpu(), want_s)
    assert s.cpu().view(torch.int32)[0, 0].item() == 0x2720D7C5
    # finer groups never quantise worse than whole rows
    qr, sr = f8.scale(x.cuda(), rt.row_amax(x).cuda())
    deq = lambda qq, ss: qq.cpu().float() * rt.tile_broadcast(ss.cpu(), x.shape)
    assert rel_l2(deq(q, s), x.float()) <= rel_l2(deq(qr, sr), x.float()) * 1.02


@pytest.mark.parametrize("mkn,g", [((40, 96, 24), 2), ((130, 1024, 200), 4), ((257, 2048, 513), 8)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_matmul_with_column_groups(mkn, g, with_bias):
    from lingua_amd import float8 as f8
    M, K, N = mkn
    a = seeded_bf16((M, K), std=1.5, seed=M)
    b_t = seeded_bf16((N, K), std=0.05, seed=N)
    a[3, K // g: 2 * K // g] *= 50.0
    bias = seeded_bf16((N,), std=0.5, seed=7) if with_bias else None
    am_a, am_b = rt.subrow_amax(a, g), rt.subrow_amax(b_t, g)
    got = f8.matmul(a.cuda(), am_a.cuda(), b_t.cuda(), am_b.cuda(), bias.cuda() if with_bias else None)
    want = rt.matmul(a, am_a, b_t, am_b, bias)
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    assert rel_l2(got, want) <= 1e-3, rel_l2(got, want)
    # and it is a better product than whole-row scaling when a group holds outliers
    exact = a.double() @ b_t.double().t() + (bias.double() if with_bias else 0.0)
    rowwise = f8.matmul(a.cuda(), rt.row_amax(a).cuda(), b_t.cuda(), rt.row_amax(b_t).cuda(), bias.cuda() if with_bias else None)
    assert rel_l2(got.double().cpu(), exact) <= rel_l2(rowwise.double().cpu(), exact) * 1.05


def test_rejected_tilings():
    from lingua_amd import float8 as f8
    x = seeded_bf16((8, 96)).cuda()
    with pytest.raises(RuntimeError, match="groups"):
        f8.scale(x, torch.ones(8, 4, device="cuda"))          # 24 columns per group: not a multiple of 16
    with pytest.raises(RuntimeError, match="groups"):
        f8.scale(x, torch.ones(8, 5, device="cuda"))          # does not divide
    with pytest.raises(RuntimeError, match="unsupported amax shape"):
        f8.scale(x, torch.ones(4, 1, device="cuda"))          # row blocks other than 1 and R
    with pytest.raises(RuntimeError, match="unsupported amax shape"):
        f8.scale(x, torch.ones(1, 2, device="cuda"))
    with pytest.raises(RuntimeError, match="column groups"):
        f8.matmul(x, torch.ones(8, 2, device="cuda"), x, torch.ones(8, 3, device="cuda"), None)


def test_scale_uses_the_row_amax_it_is_given():
    """scale(t, amax [R,1]) multiplies by 448 / amax of the ARGUMENT (lingua/float8.py:43-47): the true amax gives the
    fused kernel's bytes, a repeated tensor amax (what lingua/float8.py:115-118 builds) gives the tensor-wise bytes,
    and an amax below the true one saturates / overflows as the ATen cast does."""
    from golden_util import fp8_equal_mod_nan_sign
    from lingua_amd import float8 as f8, ops
    x = seeded_bf16((300, 1024), std=2.0, seed=77)
    x[5] = 0.0
    x[7, 100] = 3000.0
    xd = x.cuda()
    true_amax = rt.row_amax(x)
    # (1) the true amax: same bytes and scales as the fused kernel and as the oracle
    q, s = f8.scale(xd, true_amax.cuda())
    qf, sf, _ = ops.cast_rowwise(xd)
    qo, so, _ = oracle.cast_rowwise(x)
    assert torch.equal(q.view(torch.uint8), qf.view(torch.uint8)) and bits_equal(s, sf)
    assert torch.equal(q.cpu().view(torch.uint8), qo) and bits_equal(s.cpu().reshape(-1), so)
    # (2) every row holds the tensor amax: the tensor-wise quantisation
    rep = true_amax.amax().reshape(1, 1).repeat(300, 1)
    q2, s2 = f8.scale(xd, rep.cuda())
    qt, st_ = oracle.cast_tensorwise(x)
    assert torch.equal(q2.cpu().view(torch.uint8), qt)
    assert bits_equal(s2.cpu().reshape(-1), st_.repeat(300))
    # (3) an amax that is too small (a quarter of the true one), a negative one and a zero one: the PyTorch op chain
    wrong = (true_amax.float() / 4).to(torch.bfloat16)
    wrong[9] = -1.0
    wrong[11] = 0.0
    q3, s3 = f8.scale(xd, wrong.cuda())
    want_q, want_s = rt.scale(x, wrong)
    assert fp8_equal_mod_nan_sign(q3, want_q) and bits_equal(s3.cpu(), want_s)
    codes = q3.cpu().view(torch.uint8) & 0x7F
    assert (codes == 0x7F).any() and (codes == 0x7E).any()       # both the NaN code and the clipped 448 occur
    # (4) non-finite amaxes
    bad = true_amax.clone()
    bad[1], bad[2] = float("inf"), float("nan")
    q4, s4 = f8.scale(xd, bad.cuda())
    want_q, want_s = rt.scale(x, bad)
    assert fp8_equal_mod_nan_sign(q4, want_q) and bits_equal(s4.cpu(), want_s)
    # (5) an fp32 amax that is not a bf16 value (a history of amaxes, a margin): the reference converts with
    # .float() (lingua/float8.py:44), so no bit of it may be lost; row-wise and tensor-wise
    amax32 = true_amax.float() * 1.003 + 1e-3
    assert not torch.equal(amax32.to(torch.bfloat16).float(), amax32)
    q5, s5 = f8.scale(xd, amax32.cuda())
    want_q, want_s = rt.scale(x, amax32)
    assert torch.equal(q5.cpu().view(torch.uint8), want_q.view(torch.uint8)) and bits_equal(s5.cpu(), want_s)
    t32 = (amax32.amax() * 1.01).reshape(1, 1)
    q6, s6 = f8.scale(xd, t32.cuda())
    want_q, want_s = rt.scale(x, t32)
    assert torch.equal(q6.cpu().view(torch.uint8), want_q.view(torch.uint8)) and bits_equal(s6.cpu().reshape(-1), want_s.reshape(-1))
    # fp16 goes through fp32, exactly as .float() would take it
    q7, s7 = f8.scale(xd, amax32.half().cuda())
    want_q, want_s = rt.scale(x, amax32.half())
    assert torch.equal(q7.cpu().view(torch.uint8), want_q.view(torch.uint8)) and bits_equal(s7.cpu(), want_s)


def test_matmul_called_as_the_reference_dgrad_calls_it():
    """lingua/float8.py:110-119: grad_out with its row amax, the transposed weight with its tensor amax repeated
    over the rows.  The public matmul() must honour that amax and give the oracle's dgrad."""
    from lingua_amd import float8 as f8
    M, K, N = 200, 256, 384
    g = seeded_bf16((M, N), std=1e-2, seed=5)
    w = seeded_bf16((N, K), std=0.02, seed=6)
    w[3, 10] = 1.0                                             # one large weight: row-wise and tensor-wise differ
    b = w.t().contiguous()                                     # [K,N], what lingua/float8.py:111 makes
    amax_b = rt.tensor_amax_from_rows(rt.row_amax(w), K)       # [K,1], every row the tensor amax
    got = f8.matmul(g.cuda(), rt.row_amax(g).cuda(), b.cuda(), amax_b.cuda(), None, use_fast_accum=False)
    assert rel_l2(got, oracle.linear_dgrad(g, w)) <= 1e-3
    rowwise_b = f8.matmul(g.cuda(), rt.row_amax(g).cuda(), b.cuda(), rt.row_amax(b).cuda(), None)
    assert not torch.equal(got, rowwise_b)
