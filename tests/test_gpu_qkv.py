"""GPU tests of the single product for the attention projections (lingua/transformer.py:357-359 under
lingua_amd.qkv.fuse_qkv): same bits as three separate Fp8Linear products, one GEMM launch in forward, and the
right thing when the three linears are not called the way the reference's attention calls them."""
import copy

import pytest
import torch

from conftest import rel_l2, seeded_bf16
import bench_workloads as workloads

pytestmark = pytest.mark.gpu


class Projections(torch.nn.Module):
    def __init__(self, dim, nq, nkv):
        super().__init__()
        self.wq = torch.nn.Linear(dim, nq, bias=False)
        self.wk = torch.nn.Linear(dim, nkv, bias=False)
        self.wv = torch.nn.Linear(dim, nkv, bias=False)

    def forward(self, x):
        return self.wq(x.view_as(x)), self.wk(x.view_as(x)), self.wv(x.view_as(x))


def make(dim=256, nq=512, nkv=128):
    from lingua_amd import convert_linears_to_fp8
    torch.manual_seed(11)
    root = torch.nn.ModuleDict({"attention": Projections(dim, nq, nkv)}).cuda().to(torch.bfloat16)
    return convert_linears_to_fp8(root, "rowwise", "attention")


def run(root, x, gs):
    x = x.clone().requires_grad_(True)
    for p in root.parameters():
        p.grad = None
    outs = root["attention"](x)
    torch.autograd.backward(outs, gs)
    att = root["attention"]
    return [o.detach() for o in outs], x.grad, [att.wq.weight.grad, att.wk.weight.grad, att.wv.weight.grad]


def test_one_product_same_bits_as_three():
    from lingua_amd import ops
    from lingua_amd.qkv import fuse_qkv
    plain = make()
    fused = fuse_qkv(copy.deepcopy(plain))
    assert list(fused.state_dict()) == list(plain.state_dict())
    x = seeded_bf16((3, 50, 256), seed=40).cuda()
    gs = [seeded_bf16((3, 50, n), std=0.02, seed=41 + i).cuda() for i, n in enumerate((512, 128, 128))]
    rec = []
    ops.kernel_timer = rec
    try:
        o_f, gx_f, gw_f = run(fused, x, gs)
        n_gemm_fused = sum(1 for r in rec if r[0] == "gemm_nt")
        del rec[:]
        o_p, gx_p, gw_p = run(plain, x, gs)
        n_gemm_plain = sum(1 for r in rec if r[0] == "gemm_nt")
    finally:
        ops.kernel_timer = None
    assert n_gemm_plain == 9 and n_gemm_fused == 7   # forward 3 -> 1; three dgrads and three wgrads either way
    for a, b in zip(o_f + gw_f, o_p + gw_p):
        assert a.shape == b.shape and torch.equal(a, b)
    # dX: the same three dgrads, added in the order q, k, v (autograd's own order for the plain model differs, and
    # bf16 additions do not associate): rebuild it from the plain model's three dgrads taken one at a time
    parts = []
    for i in range(3):
        xi = x.clone().requires_grad_(True)
        plain["attention"](xi)[i].backward(gs[i])
        parts.append(xi.grad)
    assert torch.equal(gx_f, (parts[0] + parts[1]) + parts[2])
    assert rel_l2(gx_f, gx_p) <= 5e-3


def test_other_call_patterns_still_compute_each_product():
    from lingua_amd.qkv import fuse_qkv
    plain = make()
    fused = fuse_qkv(copy.deepcopy(plain))
    pa, fa = plain["attention"], fused["attention"]
    x = seeded_bf16((40, 256), seed=50).cuda()
    z = seeded_bf16((40, 256), seed=51).cuda()
    with torch.no_grad():
        assert torch.equal(fa.wk(x), pa.wk(x))                    # wk before any wq
        q = fa.wq(x)
        assert torch.equal(fa.wk(z), pa.wk(z))                    # another tensor: own product, nothing stale
        assert torch.equal(fa.wv(x), pa.wv(x)) and torch.equal(q, pa.wq(x))
        fa.wq(x)
        x.mul_(0.5)                                               # changed in place between wq and wk
        assert torch.equal(fa.wk(x), pa.wk(x))
    with torch.inference_mode():
        xi = seeded_bf16((40, 256), seed=52).cuda()
        assert torch.equal(fa.wq(xi), pa.wq(xi)) and torch.equal(fa.wv(xi), pa.wv(xi))


def test_rejects_modules_that_are_not_converted_projections():
    from lingua_amd.qkv import fuse_qkv
    root = torch.nn.ModuleDict({"attention": Projections(64, 64, 64)})
    with pytest.raises(RuntimeError):
        fuse_qkv(root)


def test_llama_step_with_fused_projections_matches_drop_in():
    from lingua_amd import convert_linears_to_fp8
    from lingua_amd.norm import fuse_rmsnorm
    from lingua_amd.qkv import fuse_qkv
    torch.manual_seed(3)
    base = workloads.Llama(2, 256, 4, 512, 1000).cuda().to(torch.bfloat16)
    drop = convert_linears_to_fp8(copy.deepcopy(base), "rowwise", r"layers\.[0-9]+\.")
    fused = fuse_qkv(fuse_rmsnorm(convert_linears_to_fp8(copy.deepcopy(base), "rowwise", r"layers\.[0-9]+\.")))
    tok = torch.randint(0, 1000, (2, 64), device="cuda")
    losses = []
    for m in (drop, fused):
        logits = m(tok)
        loss = torch.nn.functional.cross_entropy(logits.float().flatten(0, 1), tok.flatten())
        loss.backward()
        losses.append(loss.item())
    assert abs(losses[0] - losses[1]) <= 2e-2 * abs(losses[0])
    for (n, a), (_, b) in zip(drop.named_parameters(), fused.named_parameters()):
        assert rel_l2(a.grad, b.grad) <= 3e-2, n
