"""GPU parity of the drop-in module / autograd function against the oracle's
three products (forward, dgrad, wgrad) and the reference interface behaviour."""
import pytest
import torch
from torch import nn

import oracle
from oracle import recipe_torch as rt
from conftest import rel_l2, seeded_bf16
from golden_util import load_golden

pytestmark = pytest.mark.gpu

TOL = 1e-3


def run_fn(x, w, go, bias=None, x_grad=True, w_grad=True):
    from lingua_amd.float8 import Fp8LinearFn
    xd = x.cuda().requires_grad_(x_grad)
    wd = w.cuda().requires_grad_(w_grad)
    bd = bias.cuda().requires_grad_(True) if bias is not None else None
    y = Fp8LinearFn.apply(xd, wd, bd)
    y.backward(go.cuda())
    return y.detach(), xd.grad, wd.grad, (bd.grad if bd is not None else None)


def test_golden_forward_backward():
    g = load_golden()
    y, dx, dw, db = run_fn(g["x_prod"], g["w"], g["go"], g["bias"])
    assert rel_l2(y, g["y"]) <= TOL
    assert rel_l2(dx, g["dx"]) <= TOL
    assert rel_l2(dw, g["dw_fp8"]) <= TOL
    assert rel_l2(db, g["go"].float().sum(0)) <= 5e-3
    assert y.dtype == dx.dtype == dw.dtype == torch.bfloat16


def test_reference_bf16_wgrad_option():
    from lingua_amd import float8
    g = load_golden()
    float8.config.fp8_wgrad = False
    try:
        y, dx, dw, _ = run_fn(g["x_prod"], g["w"], g["go"])
    finally:
        float8.config.fp8_wgrad = True
    assert rel_l2(dw, g["dw_bf16"]) <= 5e-3
    assert rel_l2(dx, g["dx"]) <= TOL


def test_grads_are_none_where_not_required():
    g = load_golden()
    _, dx, dw, _ = run_fn(g["x_prod"], g["w"], g["go"], x_grad=False)
    assert dx is None and rel_l2(dw, g["dw_fp8"]) <= TOL
    _, dx, dw, _ = run_fn(g["x_prod"], g["w"], g["go"], w_grad=False)
    assert dw is None and rel_l2(dx, g["dx"]) <= TOL


@pytest.mark.parametrize("mkn", [(512, 256, 384), (1000, 272, 144), (77, 64, 48), (2048, 1024, 4096)])
def test_three_products_vs_oracle(mkn):
    M, K, N = mkn
    x = seeded_bf16((M, K), 1.0, seed=1)
    w = seeded_bf16((N, K), 0.02, seed=2)
    go = seeded_bf16((M, N), 1e-2, seed=3)
    y, dx, dw, _ = run_fn(x, w, go)
    assert rel_l2(y, oracle.linear_forward(x, w)) <= TOL
    assert rel_l2(dx, oracle.linear_dgrad(go, w)) <= TOL
    assert rel_l2(dw, oracle.linear_wgrad_fp8(go, x)) <= TOL


def test_config1_forward_and_module_surface():
    from lingua_amd import convert_linears_to_fp8, Fp8Linear
    x = seeded_bf16((4096, 2048), 1.0, seed=0)
    w = seeded_bf16((2048, 2048), 0.02, seed=1)
    lin = nn.Linear(2048, 2048, bias=False, dtype=torch.bfloat16, device="cuda")
    with torch.no_grad():
        lin.weight.copy_(w)
    m = convert_linears_to_fp8(nn.Sequential(lin), "rowwise", "")
    assert type(m[0]) is Fp8Linear and m[0].weight is lin.weight
    y = m(x.cuda().reshape(8, 512, 2048))                     # any-rank input: flattened, then restored
    assert y.shape == (8, 512, 2048) and y.dtype == torch.bfloat16
    want = oracle.linear_forward(x, w)
    assert rel_l2(y.reshape(4096, 2048), want) <= TOL
    # the torch-op restatement agrees too (the figure the benchmark's CPU baseline times)
    assert rel_l2(y.reshape(4096, 2048), rt.linear_forward(x, w)) <= TOL


class SwiGLU(nn.Module):
    """SwiGLU feed-forward with the layer names of lingua/transformer.py:430-471."""

    def __init__(self, dim, hidden):
        super().__init__()
        self.w1 = nn.Linear(dim, hidden, bias=False)
        self.w3 = nn.Linear(dim, hidden, bias=False)
        self.w2 = nn.Linear(hidden, dim, bias=False)

    def forward(self, x):
        return self.w2(torch.nn.functional.silu(self.w1(x)) * self.w3(x))


def make_mlp(dim, hidden, seed):
    from lingua_amd import convert_linears_to_fp8
    g = torch.Generator().manual_seed(seed)
    m = SwiGLU(dim, hidden).to(torch.bfloat16)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).to(torch.bfloat16))
    cpu_w = {k: v.detach().clone() for k, v in m.state_dict().items()}
    layers = nn.ModuleDict({"layers": nn.ModuleList([m])})    # dotted names "layers.0.w1" as the default filter expects
    layers = convert_linears_to_fp8(layers.cuda(), "rowwise", r"layers\.[0-9]+\.")
    return layers["layers"][0], cpu_w


def capture_linears(mlp, names=("w1", "w3", "w2")):
    """Hooks that record, per linear, what it saw: input and output in forward, grad_out and grad_in in backward."""
    seen, hooks = {}, []
    for name in names:
        lin = getattr(mlp, name)
        hooks.append(lin.register_forward_hook(
            lambda m_, inp, out, name=name: seen.__setitem__(name + ":io", (inp[0].detach(), out.detach()))))
        hooks.append(lin.register_full_backward_hook(
            lambda m_, gin, gout, name=name: seen.__setitem__(name + ":g", (gin[0].detach() if gin[0] is not None else None,
                                                                           gout[0].detach()))))
    return seen, hooks


def test_config2_1b_mlp_forward_rows_vs_oracle():
    # rows of a row-wise-scaled forward are independent: a sample of token rows pins the full-size result.  Every
    # linear is compared with the oracle on the input the GPU handed it, so each product is held to TOL by itself.
    dim, hidden, tokens = 2048, 8192, 32768
    mlp, w = make_mlp(dim, hidden, seed=0)
    x = seeded_bf16((tokens, dim), 1.0, seed=0)
    seen, hooks = capture_linears(mlp)
    with torch.no_grad():
        y = mlp(x.cuda().reshape(8, 4096, dim)).reshape(tokens, dim)
    for h_ in hooks:
        h_.remove()
    rows = torch.arange(0, tokens, tokens // 32)[:32]
    for name in ("w1", "w3", "w2"):
        a_in, out = (t.reshape(tokens, -1) for t in seen[name + ":io"])
        assert rel_l2(out[rows.cuda()], oracle.linear_forward(a_in[rows.cuda()].cpu(), w[name + ".weight"])) <= TOL, name
    assert torch.equal(seen["w1:io"][0].reshape(tokens, dim).cpu(), x)
    # the gate between the products is PyTorch's: w2's input is silu(w1 out) * (w3 out), bit for bit
    gate = torch.nn.functional.silu(seen["w1:io"][1]) * seen["w3:io"][1]
    assert torch.equal(gate, seen["w2:io"][0])
    assert torch.equal(seen["w2:io"][1].reshape(tokens, dim), y)
    # and the chain as a whole against the oracle's own chain (three bf16 roundings deep)
    xs = x[rows]
    h = torch.nn.functional.silu(oracle.linear_forward(xs, w["w1.weight"])) * oracle.linear_forward(xs, w["w3.weight"])
    assert rel_l2(y[rows.cuda()], oracle.linear_forward(h, w["w2.weight"])) <= 3 * TOL


def test_config3_7b_mlp_forward_backward():
    # y, dX, dW1, dW2, dW3 of the 7B MLP at full size.  Each of the three linears is compared with the oracle on the
    # operands the GPU handed it (captured by hooks): forward and dgrad on a sample of token rows (rows are
    # independent under row-wise scaling), wgrad on a sample of output rows x input columns (its reduction runs over
    # every token), each within TOL.
    dim, hidden, tokens = 4096, 11008, 16384
    mlp, w = make_mlp(dim, hidden, seed=0)
    x = seeded_bf16((tokens, dim), 1.0, seed=0)
    gy = seeded_bf16((tokens, dim), 1e-2, seed=1)
    xd = x.cuda().requires_grad_(True)
    seen, hooks = capture_linears(mlp)
    y = mlp(xd)
    y.backward(gy.cuda())
    for h_ in hooks:
        h_.remove()
    rows = torch.arange(0, tokens, tokens // 24)[:24]
    rows_d = rows.cuda()
    dx_parts = {}
    for name in ("w1", "w3", "w2"):
        W = w[name + ".weight"]
        a_in, out = (t.reshape(tokens, -1) for t in seen[name + ":io"])
        g_in, g_out = (t.reshape(tokens, -1) for t in seen[name + ":g"])
        lin = getattr(mlp, name)
        assert rel_l2(out[rows_d], oracle.linear_forward(a_in[rows_d].cpu(), W)) <= TOL, name + " forward"
        want_dgrad = oracle.linear_dgrad(g_out[rows_d].cpu(), W)
        assert rel_l2(g_in[rows_d], want_dgrad) <= TOL, name + " dgrad"
        dx_parts[name] = want_dgrad
        n_idx = torch.arange(0, W.shape[0], max(1, W.shape[0] // 40))[:40]
        k_idx = torch.arange(0, W.shape[1], max(1, W.shape[1] // 40))[:40]
        qg, sg = oracle.cast_colwise_transposed(g_out[:, n_idx.cuda()].cpu())
        qa, sa = oracle.cast_colwise_transposed(a_in[:, k_idx.cuda()].cpu())
        want_dw = oracle.gemm_nt(qg, qa, sg, sa)
        got_dw = lin.weight.grad[n_idx.cuda()][:, k_idx.cuda()]
        assert rel_l2(got_dw, want_dw) <= TOL, name + " wgrad"
    # what the linears were handed is what the module saw: x, the gate, gy
    assert torch.equal(seen["w1:io"][0].cpu(), x) and torch.equal(seen["w3:io"][0].cpu(), x)
    assert torch.equal(seen["w2:g"][1].cpu(), gy) and torch.equal(seen["w2:io"][1], y.detach())
    # dX = dgrad(w1) + dgrad(w3), added by autograd in bf16
    want_dx = (dx_parts["w1"].float() + dx_parts["w3"].float()).to(torch.bfloat16)
    assert xd.grad.shape == x.shape and xd.grad.dtype == torch.bfloat16
    assert rel_l2(xd.grad[rows_d], want_dx) <= TOL
    assert torch.isfinite(xd.grad.float()).all()
    # y against the oracle's own chain (three bf16 roundings deep)
    xs = x[rows]
    hh = torch.nn.functional.silu(oracle.linear_forward(xs, w["w1.weight"])) * oracle.linear_forward(xs, w["w3.weight"])
    assert rel_l2(y.detach()[rows_d], oracle.linear_forward(hh, w["w2.weight"])) <= 3 * TOL


def test_outlier_stress_rowwise_beats_tensorwise_on_the_linear():
    # config 4 at its full 16384 tokens: both recipes against the oracle's product of the very same bytes and scales
    # on a row sample, then the two recipes against each other
    from bench_workloads import outlier_stress_figures
    fig, t = outlier_stress_figures(16384)
    rows = torch.arange(0, 16384, 512).cuda()
    want_row = oracle.gemm_nt(t["qx"][rows].cpu().view(torch.uint8), t["qw"].cpu().view(torch.uint8), t["sx"][rows].cpu(), t["sw"].cpu())
    want_ten = oracle.gemm_nt(t["qxt"][rows].cpu().view(torch.uint8), t["qwt"].cpu().view(torch.uint8), t["sxt"].cpu(), t["swt"].cpu())
    assert rel_l2(t["y_row"][rows], want_row) <= TOL
    assert rel_l2(t["y_ten"][rows], want_ten) <= TOL
    # and against the oracle's whole row-wise linear from the bf16 operands
    assert rel_l2(t["y_row"][rows], oracle.linear_forward(t["x"][rows.cpu()], t["w"])) <= TOL
    print("config 4:", fig)
    assert fig["rel_l2_y_rowwise"] < fig["rel_l2_y_tensorwise"]
    assert fig["snr_x_rowwise_db"] > fig["snr_x_tensorwise_db"]
    assert (t["y_row"][t["zero_rows"].cuda()] == 0).all()        # all-zero token rows give exact zeros


def test_config5_llama_1b_training_step():
    # full Llama-1B-shaped step (25 layers, dim 2048, 16 heads, ffn 8192, vocab 128256, 4 x 4096 tokens), all block
    # linears fp8 row-wise, output head bf16; three linears are checked against the oracle through hooks
    from lingua_amd import convert_linears_to_fp8, Fp8Linear
    from bench_workloads import Llama, LLAMA_1B
    torch.manual_seed(0)
    with torch.device("cuda"):
        model = Llama(**LLAMA_1B).to(torch.bfloat16)
    model.init_weights(0.02, seed=0)
    g = torch.Generator().manual_seed(0)
    tokens = torch.randint(0, LLAMA_1B["vocab"], (4, 4096), generator=g).cuda()
    labels = torch.randint(0, LLAMA_1B["vocab"], (4, 4096), generator=g).cuda()
    with torch.no_grad():
        loss_bf16 = float(model(tokens, labels))
    keys_before = list(model.state_dict().keys())
    model = convert_linears_to_fp8(model, "rowwise", r"layers\.[0-9]+\.")
    n_fp8 = sum(1 for m in model.modules() if type(m) is Fp8Linear)
    assert n_fp8 == 25 * 7
    assert type(model.output) is nn.Linear and list(model.state_dict().keys()) == keys_before

    picks = {"layers.0.attention.wq": None, "layers.12.feed_forward.w2": None, "layers.24.feed_forward.w1": None}
    seen, hooks = {}, []
    mods = dict(model.named_modules())
    for name in picks:
        m = mods[name]
        hooks.append(m.register_forward_hook(
            lambda m_, inp, out, name=name: seen.__setitem__(name + ":io", (inp[0].detach(), out.detach()))))
        hooks.append(m.register_full_backward_hook(
            lambda m_, gin, gout, name=name: seen.__setitem__(name + ":g", (gin[0].detach(), gout[0].detach()))))
    loss = model(tokens, labels)
    loss.backward()
    for h_ in hooks:
        h_.remove()
    assert torch.isfinite(loss) and abs(float(loss.detach()) - loss_bf16) < 0.05 * abs(loss_bf16)
    rows = torch.arange(0, 16384, 16384 // 16)[:16].cuda()
    for name in picks:
        lin = mods[name]
        W = lin.weight.detach().cpu()
        a_in, out = (t.flatten(0, 1) for t in seen[name + ":io"])
        g_in, g_out = (t.flatten(0, 1) for t in seen[name + ":g"])
        assert rel_l2(out[rows], oracle.linear_forward(a_in[rows].cpu(), W)) <= TOL, name
        assert rel_l2(g_in[rows], oracle.linear_dgrad(g_out[rows].cpu(), W)) <= TOL, name
        n_idx = torch.arange(0, W.shape[0], max(1, W.shape[0] // 24))[:24].cuda()
        k_idx = torch.arange(0, W.shape[1], max(1, W.shape[1] // 24))[:24].cuda()
        qg, sg = oracle.cast_colwise_transposed(g_out[:, n_idx].cpu())
        qa, sa = oracle.cast_colwise_transposed(a_in[:, k_idx].cpu())
        want = oracle.gemm_nt(qg, qa, sg, sa)
        assert rel_l2(lin.weight.grad[n_idx][:, k_idx], want) <= TOL, name
    assert all(p.grad is not None and torch.isfinite(p.grad.float()).all() for p in model.parameters())


def test_linears_on_the_same_activation_share_its_casts():
    """w1 / w3 style: the second linear on the same input reuses the quantised copy (forward and
    backward); a new pass quantises afresh; results are bit-identical with sharing off."""
    from lingua_amd import Fp8Linear, float8, ops
    torch.manual_seed(5)
    l1 = Fp8Linear(256, 512, bias=False, device="cuda", dtype=torch.bfloat16)
    l3 = Fp8Linear(256, 512, bias=False, device="cuda", dtype=torch.bfloat16)
    x = seeded_bf16((2, 40, 256), seed=21).cuda().requires_grad_(True)
    g = seeded_bf16((2, 40, 512), std=0.02, seed=22).cuda()

    def run(share):
        old = float8.config.share_input_casts
        float8.config.share_input_casts = share
        rec = []
        ops.kernel_timer = rec
        try:
            for p in (l1.weight, l3.weight, x):
                p.grad = None
            y1, y3 = l1(x), l3(x)
            n_fwd = sum(1 for r in rec if r[0] == "cast_rowwise")
            (y1 * 2 + y3).backward(g)
            n_bwd_t = sum(1 for r in rec if r[0] == "cast_colwise_t")
            # a second forward over the same tensor is a new pass: the activation is quantised again
            del rec[:]
            with torch.no_grad():
                l1(x), l3(x)
            n_again = sum(1 for r in rec if r[0] == "cast_rowwise")
        finally:
            ops.kernel_timer = None
            float8.config.share_input_casts = old
        return (y1.detach(), y3.detach(), x.grad.clone(), l1.weight.grad.clone(), l3.weight.grad.clone()), (n_fwd, n_bwd_t, n_again)

    shared, counts_shared = run(True)
    apart, counts_apart = run(False)
    assert counts_apart == (4, 4, 4), counts_apart     # x twice + two weights; two grads + x twice
    assert counts_shared == (3, 3, 3), counts_shared   # x once per pass
    for a, b in zip(shared, apart):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    # an in-place change of the activation is seen (version counter)
    with torch.no_grad():
        ya = l1(x)
        x.mul_(2.0)
        yb = l3(x)
        yc = l3(x / 1.0)
    assert torch.equal(yb, yc) and not torch.equal(ya, yb)


def test_custom_ops_route_equals_the_autograd_function_and_compiles():
    """config.use_custom_ops: same bits as the plain autograd.Function; the converted model traces as one graph
    (aot_eager: fake tensors + functionalisation + the registered autograd formula, no code generation)."""
    from lingua_amd import convert_linears_to_fp8, float8
    from lingua_amd import custom_ops
    from bench_workloads import FeedForward
    torch.manual_seed(6)
    holder = nn.ModuleDict({"feed_forward": FeedForward(256, 512).to(device="cuda", dtype=torch.bfloat16)})
    model = convert_linears_to_fp8(holder, "rowwise", r"feed_forward\.")["feed_forward"]
    x = seeded_bf16((3, 32, 256), seed=31).cuda()
    gy = seeded_bf16((3, 32, 256), std=0.02, seed=32).cuda()

    def run(fn):
        for p in model.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        y = fn(xi)
        y.backward(gy)
        return [y.detach(), xi.grad] + [p.grad.clone() for p in model.parameters()]

    want = run(model)
    old = float8.config.use_custom_ops
    float8.config.use_custom_ops = True
    try:
        got = run(model)
        compiled = torch.compile(model, backend="aot_eager", fullgraph=True)
        got_compiled = run(compiled)
        # the operators are addressable by name (what a checkpointing policy lists)
        assert torch.ops.lingua_amd.fp8_linear_fwd.default is not None
        torch.library.opcheck(custom_ops.fp8_linear_fwd, (x.flatten(0, 1), model.w1.weight.detach(), None, True, 0),
                              test_utils=("test_schema", "test_faketensor"))
    finally:
        float8.config.use_custom_ops = old
    for a, b in zip(got, want):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for a, b in zip(got_compiled, want):
        assert rel_l2(a, b) <= 1e-6


def test_empty_batch_and_single_token():
    """Zero tokens (an empty micro-batch) and one token go through forward and backward: outputs of the right
    shape, zero weight gradient for the empty batch, oracle parity for the single token."""
    from lingua_amd import Fp8Linear
    torch.manual_seed(8)
    lin = Fp8Linear(128, 256, bias=True, device="cuda", dtype=torch.bfloat16)
    x0 = torch.zeros((0, 128), dtype=torch.bfloat16, device="cuda", requires_grad=True)
    y0 = lin(x0)
    assert y0.shape == (0, 256)
    y0.backward(torch.zeros_like(y0))
    assert x0.grad.shape == (0, 128)
    assert float(lin.weight.grad.float().abs().max()) == 0.0 and float(lin.bias.grad.float().abs().max()) == 0.0
    lin.weight.grad = lin.bias.grad = None
    x1 = seeded_bf16((1, 128), seed=41).cuda().requires_grad_(True)
    g1 = seeded_bf16((1, 256), std=0.02, seed=42).cuda()
    y1 = lin(x1)
    y1.backward(g1)
    W, b = lin.weight.detach().cpu(), lin.bias.detach().cpu()
    assert rel_l2(y1, oracle.linear_forward(x1.detach().cpu(), W, b)) <= TOL
    assert rel_l2(x1.grad, oracle.linear_dgrad(g1.cpu(), W)) <= TOL
    assert rel_l2(lin.weight.grad, oracle.linear_wgrad_fp8(g1.cpu(), x1.detach().cpu())) <= TOL
    assert torch.equal(lin.bias.grad, g1[0])


def test_mlp_step_is_bitwise_reproducible():
    """No result of the path depends on scheduling: the column amaxes are max-merged (order-free), every sum runs
    in a fixed order.  Two runs of the same MLP step give identical bits, drop-in and fused."""
    from lingua_amd import convert_linears_to_fp8
    from bench_workloads import FeedForward
    from lingua_amd.swiglu import Fp8FeedForward
    torch.manual_seed(12)
    holder = nn.ModuleDict({"feed_forward": FeedForward(512, 1536).to(device="cuda", dtype=torch.bfloat16)})
    mlp = convert_linears_to_fp8(holder, "rowwise", r"feed_forward\.")["feed_forward"]
    fused = Fp8FeedForward(mlp.w1, mlp.w3, mlp.w2)
    x = seeded_bf16((1000, 512), seed=51).cuda()
    gy = seeded_bf16((1000, 512), std=0.02, seed=52).cuda()
    for module in (mlp, fused):
        runs = []
        for _ in range(2):
            for p in module.parameters():
                p.grad = None
            xi = x.clone().requires_grad_(True)
            y = module(xi)
            y.backward(gy)
            runs.append([y.detach(), xi.grad] + [p.grad.clone() for p in module.parameters()])
        for a, b in zip(*runs):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_fp8_copy_of_the_input_kept_for_wgrad_instead_of_the_bf16_input():
    """config.save_fp8_input: forward keeps the input quantised along the token dimension (e4m3 [K,M] + K scales)
    and not the bf16 input; same kernels on the same data, so every result is bit-identical; two linears on one
    activation share that copy; the bytes held by the graph between forward and backward drop."""
    from lingua_amd import Fp8Linear, float8, ops
    torch.manual_seed(6)
    l1 = Fp8Linear(512, 1024, bias=True, device="cuda", dtype=torch.bfloat16)
    l3 = Fp8Linear(512, 256, bias=False, device="cuda", dtype=torch.bfloat16)
    x = seeded_bf16((3, 100, 512), seed=23).cuda().requires_grad_(True)      # 300 tokens: padded to 304 in the [K,M] copy
    g1 = seeded_bf16((3, 100, 1024), std=0.02, seed=24).cuda()
    g3 = seeded_bf16((3, 100, 256), std=0.02, seed=25).cuda()

    def run(lean):
        old = float8.config.save_fp8_input
        float8.config.save_fp8_input = lean
        kept, rec = [], []
        ops.kernel_timer = rec
        try:
            for p in (l1.weight, l1.bias, l3.weight, x):
                p.grad = None
            with torch.autograd.graph.saved_tensors_hooks(lambda t: (kept.append((t.dtype, tuple(t.shape))), t)[1], lambda t: t):
                y1, y3 = l1(x), l3(x)
            n_t_fwd = sum(1 for r in rec if r[0] == "cast_colwise_t")
            torch.autograd.backward((y1, y3), (g1, g3))
            n_t_all = sum(1 for r in rec if r[0] == "cast_colwise_t")
        finally:
            ops.kernel_timer = None
            float8.config.save_fp8_input = old
        outs = [y1.detach(), y3.detach(), x.grad.clone(), l1.weight.grad.clone(), l1.bias.grad.clone(), l3.weight.grad.clone()]
        return outs, kept, (n_t_fwd, n_t_all)

    plain, kept_plain, n_plain = run(False)
    lean, kept_lean, n_lean = run(True)
    for a, b in zip(lean, plain):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    assert (torch.bfloat16, (300, 512)) in kept_plain
    assert (torch.bfloat16, (300, 512)) not in kept_lean
    assert kept_lean.count((torch.float8_e4m3fn, (512, 304))) == 2          # one shared copy, saved by both linears
    assert n_plain == (0, 3) and n_lean == (1, 3)                             # x once (forward) + the two grads
    # without fp8 wgrad, or when the weight does not learn, there is nothing to keep in fp8
    old = (float8.config.save_fp8_input, float8.config.fp8_wgrad)
    float8.config.save_fp8_input, float8.config.fp8_wgrad = True, False
    try:
        x.grad = l3.weight.grad = None
        l3(x).backward(g3)
        assert rel_l2(l3.weight.grad, plain[5]) < 5e-2
    finally:
        float8.config.save_fp8_input, float8.config.fp8_wgrad = old


def test_inference_mode_matches_no_grad():
    """Activations made under torch.inference_mode() have no version counter (apps/main/generate.py:322 of the
    reference generates that way): the shared-cast memo must step aside, results equal the no_grad ones."""
    from lingua_amd import convert_linears_to_fp8
    from lingua_amd.norm import fuse_rmsnorm
    from bench_workloads import TransformerBlock, rope_tables
    torch.manual_seed(3)
    holder = nn.ModuleDict({"layers": nn.ModuleList([TransformerBlock(256, 4, 64, 512).to(device="cuda", dtype=torch.bfloat16)])})
    x = seeded_bf16((2, 48, 256), seed=61).cuda()
    cos, sin = rope_tables(64, 48, 10000.0, x.device)
    for fuse in (False, True):
        model = convert_linears_to_fp8(holder, "rowwise", r"layers\.[0-9]+\.") if not fuse else fuse_rmsnorm(holder)
        block = model["layers"][0]
        with torch.no_grad():
            want = block(x, cos, sin)
        with torch.inference_mode():
            xi = x * 1.0                                        # an inference tensor
            assert xi.is_inference()
            got = block(xi, cos, sin)
            got2 = block(xi, cos, sin)
        assert torch.equal(got, want) and torch.equal(got2, want)


def test_raw_pointer_writes_are_seen_by_the_shared_casts():
    """A kernel of this library that writes into a caller's tensor through data_ptr() advances its version counter,
    so a linear applied afterwards does not reuse the quantised copy made before the write; writes that bypass the
    counter (.data) are the caller's to announce with clear_cast_memos()."""
    from lingua_amd import Fp8Linear, float8, ops
    torch.manual_seed(9)
    l1 = Fp8Linear(256, 256, bias=False, device="cuda", dtype=torch.bfloat16)
    l3 = Fp8Linear(256, 256, bias=False, device="cuda", dtype=torch.bfloat16)
    x = seeded_bf16((64, 256), seed=71).cuda()
    other = seeded_bf16((64, 256), seed=72).cuda()
    qa, sa, _ = ops.cast_rowwise(other)
    qb, sb, _ = ops.cast_rowwise(l1.weight.detach())
    with torch.no_grad():
        l1(x)                                                   # files q(x) in the memo
        v = x._version
        ops.gemm_nt(qa, qb, sa, sb, out=x)                      # overwrites x in place, raw pointer
        assert x._version > v
        got = l3(x)
        want = l3(x.clone())
        assert torch.equal(got, want)
        # the same for a cast written into a caller's buffer
        q_user = torch.empty(64, 256, dtype=torch.float8_e4m3fn, device="cuda")
        v = q_user._version
        ops.cast_rowwise(other, out_q=q_user)
        assert q_user._version > v
        # a .data write is invisible to the version counter (to autograd's too): announce it
        l1(x)
        x.data.copy_(other)
        float8.clear_cast_memos()
        assert torch.equal(l3(x), l3(other.clone()))


def test_selective_checkpointing_saves_the_fp8_product():
    """lingua/distributed.py:43-50,467-473: selective activation checkpointing with the linear's forward operator in
    the must-save list (where the reference lists aten._scaled_mm).  The recomputation in backward must not launch
    the forward GEMMs again, and every gradient must equal the plain run bit for bit."""
    from functools import partial
    from torch.utils.checkpoint import CheckpointPolicy, checkpoint, create_selective_checkpoint_contexts
    from lingua_amd import convert_linears_to_fp8, float8, ops
    from bench_workloads import FeedForward
    torch.manual_seed(14)
    holder = nn.ModuleDict({"feed_forward": FeedForward(256, 512).to(device="cuda", dtype=torch.bfloat16)})
    mlp = convert_linears_to_fp8(holder, "rowwise", r"feed_forward\.")["feed_forward"]
    x = seeded_bf16((4, 32, 256), seed=81).cuda()
    gy = seeded_bf16((4, 32, 256), std=0.02, seed=82).cuda()
    no_recompute = {torch.ops.lingua_amd.fp8_linear_fwd.default}

    def policy(ctx, op, *args, **kwargs):                       # the shape of lingua/distributed.py's get_default_policy
        return CheckpointPolicy.MUST_SAVE if op in no_recompute else CheckpointPolicy.PREFER_RECOMPUTE

    def run(mode):
        for p in mlp.parameters():
            p.grad = None
        xi = x.clone().requires_grad_(True)
        rec = []
        ops.kernel_timer = rec
        try:
            if mode == "plain":
                y = mlp(xi)
            elif mode == "sac":
                y = checkpoint(mlp, xi, use_reentrant=False, context_fn=partial(create_selective_checkpoint_contexts, policy))
            else:                                               # full recomputation, for the count
                y = checkpoint(mlp, xi, use_reentrant=False)
            n_fwd = sum(1 for r in rec if r[0] == "gemm_nt")
            y.backward(gy)
            n_all = sum(1 for r in rec if r[0] == "gemm_nt")
        finally:
            ops.kernel_timer = None
        return [y.detach(), xi.grad] + [p.grad.clone() for p in mlp.parameters()], (n_fwd, n_all)

    old = float8.config.use_custom_ops
    float8.config.use_custom_ops = True
    try:
        plain, n_plain = run("plain")
        sac, n_sac = run("sac")
        full, n_full = run("full")
    finally:
        float8.config.use_custom_ops = old
    assert n_plain == (3, 9)                                    # 3 forward products + 3 dgrads + 3 wgrads
    assert n_sac == (3, 9), n_sac                               # nothing multiplied twice: the products were saved
    assert n_full == (3, 12), n_full                            # plain checkpointing runs the three forwards again
    for a, b in zip(sac, plain):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    for a, b in zip(full, plain):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_weight_casts_kept_between_optimizer_steps():
    """config.cache_weight_casts: micro-batches between two optimizer steps quantise each weight once (row-wise
    for forward, tensor-wise transposed for dgrad); an in-place update of the weight is seen; same bits."""
    from lingua_amd import Fp8Linear, float8, ops
    torch.manual_seed(8)
    lin = Fp8Linear(256, 384, bias=False, device="cuda", dtype=torch.bfloat16)
    xs = [seeded_bf16((48, 256), seed=30 + i).cuda().requires_grad_(True) for i in range(2)]
    g = seeded_bf16((48, 384), std=0.02, seed=33).cuda()

    def micro_batches(cache):
        old = float8.config.cache_weight_casts
        float8.config.cache_weight_casts = cache
        float8.clear_cast_memos()
        rec = []
        ops.kernel_timer = rec
        try:
            outs = []
            for x in xs:
                x.grad = None
                lin.weight.grad = None
                y = lin(x)
                y.backward(g)
                outs += [y.detach(), x.grad.clone(), lin.weight.grad.clone()]
            counts = (sum(1 for r in rec if r[0] == "cast_rowwise"), sum(1 for r in rec if r[0] == "cast_tensorwise_t"))
            del rec[:]
            with torch.no_grad():
                lin.weight.mul_(0.5)       # the optimizer step
            y = lin(xs[0])
            outs.append(y.detach())
            after_step = sum(1 for r in rec if r[0] == "cast_rowwise")
        finally:
            ops.kernel_timer = None
            float8.config.cache_weight_casts = old
            float8.clear_cast_memos()
            with torch.no_grad():
                lin.weight.mul_(2.0)
        return outs, counts, after_step

    plain, counts_plain, again_plain = micro_batches(False)
    cached, counts_cached, again_cached = micro_batches(True)
    assert counts_plain == (6, 2), counts_plain    # per micro-batch: x, W, grad row-wise; W tensor-wise transposed
    assert counts_cached == (5, 1), counts_cached  # the weight once in each layout
    assert again_plain == 2 and again_cached == 2  # a changed weight is quantised again
    for a, b in zip(plain, cached):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_large_linear_with_bias_vs_oracle():
    """nn.Linear(4096, 4096, bias=True) on 4096 tokens: 256 tiles, so forward takes the persistent kernel's bias
    instantiation; forward (lingua/float8.py:65-73 with the bias fused), dgrad and fp8 wgrad against the oracle on
    row samples, grad_bias against the oracle's column sum (lingua/float8.py:127)."""
    from lingua_amd import Fp8Linear
    M, K, N = 4096, 4096, 4096
    lin = Fp8Linear(K, N, bias=True, device="cuda", dtype=torch.bfloat16)
    w = seeded_bf16((N, K), 0.02, seed=51)
    b = seeded_bf16((N,), 2.0, seed=52)
    with torch.no_grad():
        lin.weight.copy_(w)
        lin.bias.copy_(b)
    x = seeded_bf16((M, K), 1.0, seed=53)
    go = seeded_bf16((M, N), 1e-2, seed=54)
    xd = x.cuda().requires_grad_(True)
    y = lin(xd)
    y.backward(go.cuda())
    rows = torch.arange(0, M, M // 32)[:32]
    qx, sx, _ = oracle.cast_rowwise(x[rows])
    qw, sw, _ = oracle.cast_rowwise(w)
    assert rel_l2(y[rows.cuda()], oracle.gemm_nt(qx, qw, sx, sw, b)) <= TOL
    assert rel_l2(xd.grad[rows.cuda()], oracle.linear_dgrad(go[rows], w)) <= TOL
    # wgrad reduces over all tokens: a sample of output rows (columns of grad_out) against the oracle
    cols = torch.arange(0, N, N // 24)[:24]
    assert rel_l2(lin.weight.grad[cols.cuda()], oracle.linear_wgrad_fp8(go[:, cols].contiguous(), x)) <= TOL
    assert rel_l2(lin.bias.grad, oracle.col_sum(go)) <= 5e-3


def test_weight_cast_cache_lets_go_of_a_deleted_model():
    """config.cache_weight_casts holds each weight by weak reference: deleting the model frees the weights and
    their quantised copies (device memory returns to where it was), and the cache has no slot left."""
    import gc
    from lingua_amd import Fp8Linear, float8
    float8.clear_cast_memos()
    gc.collect()
    torch.cuda.synchronize()
    base = torch.cuda.memory_allocated()
    old = float8.config.cache_weight_casts
    float8.config.cache_weight_casts = True
    try:
        model = torch.nn.Sequential(*[Fp8Linear(512, 512, bias=False, device="cuda", dtype=torch.bfloat16) for _ in range(4)])
        x = seeded_bf16((64, 512), seed=3).cuda().requires_grad_(True)
        for _ in range(2):
            model(x).sum().backward()
        assert len(float8._weight_casts.entries) == 4
        held = torch.cuda.memory_allocated() - base
        assert held >= 4 * 512 * 512 * 4          # bf16 weights + two one-byte copies each
        del model
        x.grad = None
        del x
        float8._fwd_cast.clear(); float8._bwd_cast.clear(); float8._fwd_tcast.clear()   # the activation memos only
        gc.collect()
        assert len(float8._weight_casts.entries) == 0
        assert torch.cuda.memory_allocated() == base
    finally:
        float8.config.cache_weight_casts = old
        float8.clear_cast_memos()


def test_two_streams_keep_their_own_shared_casts():
    """The memo of the last quantised activation is kept per (device, stream): linears of one model stepping on
    one stream still share their activation's cast while another model has stepped on another stream in between
    (a single process-wide entry would be evicted by it on every call)."""
    from lingua_amd import Fp8Linear, float8, ops
    torch.manual_seed(9)
    a1 = Fp8Linear(256, 256, bias=False, device="cuda", dtype=torch.bfloat16)
    a3 = Fp8Linear(256, 256, bias=False, device="cuda", dtype=torch.bfloat16)
    other = Fp8Linear(256, 256, bias=False, device="cuda", dtype=torch.bfloat16)
    x = seeded_bf16((64, 256), seed=5).cuda()
    z = seeded_bf16((64, 256), seed=6).cuda()
    side = torch.cuda.Stream()
    float8.clear_cast_memos()
    torch.cuda.synchronize()
    rec = []
    ops.kernel_timer = rec
    try:
        with torch.no_grad():
            y1 = a1(x)
            with torch.cuda.stream(side):
                other(z)                      # another model, another stream, between w1 and w3 of the first
            y3 = a3(x)
        torch.cuda.synchronize()
    finally:
        ops.kernel_timer = None
        float8.clear_cast_memos()
    # row-wise casts: x once (shared by a1 and a3), z once, three weights
    assert sum(1 for r in rec if r[0] == "cast_rowwise") == 5
    with torch.no_grad():
        float8.config.share_input_casts = False
        try:
            assert torch.equal(y1, a1(x)) and torch.equal(y3, a3(x))
        finally:
            float8.config.share_input_casts = True


@pytest.mark.parametrize("shape", [(4096, 2048, 2048, False), (2000, 1024, 4096, True)])
def test_forward_and_dgrad_against_the_reference_op_chain_run_on_this_gpu(shape, gpu_division_rule):
    """The reference's sequence of ATen ops, issued op for op by oracle.recipe_torch (abs / amax / clamp / div /
    reciprocal / mul / to(float8_e4m3fn), lingua/float8.py:43-47,86-87,115-118), run by PyTorch's own kernels on this
    GPU, with the product through torch._scaled_mm exactly as lingua/float8.py:65-73 calls it.  Under the division
    rule of PyTorch's GPU kernel (`set_scale_rule("times_inverse")`; under the default rule, the CPU kernel's, half
    the scales differ in their last bit and 0.03-0.1 % of the bytes with them) the fp8 bytes and scales of this library
    must equal that chain's bit for bit; y and dX must agree an order of magnitude inside the benchmark's tolerance
    (the two products run on the same matrix instructions)."""
    from golden_util import bits_equal
    from lingua_amd import ops
    import lingua_amd.float8 as f8
    M, K, N, with_bias = shape
    x = seeded_bf16((M, K), 1.0, seed=11).cuda()
    w = seeded_bf16((N, K), 0.02, seed=12).cuda()
    b = seeded_bf16((N,), 0.5, seed=13).cuda() if with_bias else None
    gy = seeded_bf16((M, N), 1e-2, seed=14).cuda()

    def mm(q1, s1, q2_t, s2_t, bias=None):
        return torch._scaled_mm(q1, q2_t.t(), scale_a=s1, scale_b=s2_t.t(), bias=bias, out_dtype=torch.bfloat16,
                                use_fast_accum=True)

    # forward: both operands row-wise
    qx_ref, sx_ref = rt.scale(x, rt.row_amax(x))
    qw_ref, sw_ref = rt.scale(w, rt.row_amax(w))
    qx, sx, ax = ops.cast_rowwise(x)
    qw, sw, aw = ops.cast_rowwise(w)
    assert bits_equal(qx.view(torch.uint8), qx_ref.view(torch.uint8)) and bits_equal(sx.reshape(-1), sx_ref.reshape(-1))
    assert bits_equal(qw.view(torch.uint8), qw_ref.view(torch.uint8)) and bits_equal(sw.reshape(-1), sw_ref.reshape(-1))
    assert bits_equal(ax.reshape(-1), rt.row_amax(x).reshape(-1))
    try:
        y_ref = mm(qx_ref, sx_ref, qw_ref, sw_ref, b)
    except (RuntimeError, NotImplementedError) as e:
        pytest.skip(f"torch._scaled_mm with row-wise scales is not available here: {e}")
    lin = f8.Fp8Linear(K, N, bias=with_bias, dtype=torch.bfloat16, device="cuda")
    with torch.no_grad():
        lin.weight.copy_(w)
        if with_bias:
            lin.bias.copy_(b)
    xg = x.clone().requires_grad_(True)
    y = lin(xg)
    assert rel_l2(y, y_ref) <= 1e-4
    # dgrad: grad_out row-wise, the weight with one scale for the whole tensor, transposed copy
    y.backward(gy)
    wt = w.t().contiguous()
    amax_wt = rt.tensor_amax_from_rows(rt.row_amax(w), K)
    qg_ref, sg_ref = rt.scale(gy, rt.row_amax(gy))
    qwt_ref, swt_ref = rt.scale(wt, amax_wt)
    qwt, swt = ops.cast_tensorwise(w, ops.amax_reduce(aw), transpose=True)
    assert bits_equal(qwt.view(torch.uint8), qwt_ref.view(torch.uint8))
    assert bits_equal(swt.reshape(-1), swt_ref[:1].reshape(-1))
    dx_ref = mm(qg_ref, sg_ref, qwt_ref, swt_ref)
    assert rel_l2(xg.grad, dx_ref) <= 1e-4
