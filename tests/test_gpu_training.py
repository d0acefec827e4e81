"""A short training run (AdamW on one fixed batch) of a small Llama: bf16, through convert_linears_to_fp8, and
with every opt-in on top (fused gate and norms, fp8 input copies, the torch.library route).  In-place parameter
updates between steps, repeated passes over the same module tree and the quantisation memo all come together
here; every variant must learn the batch as the bf16 model does."""
import pytest
import torch

pytestmark = pytest.mark.gpu

CFG = dict(n_layers=3, dim=256, n_heads=4, ffn_dim=768, vocab=512)
STEPS = 40


def _train(kind):
    from lingua_amd import convert_linears_to_fp8, float8
    from bench_workloads import Llama
    from lingua_amd.norm import fuse_rmsnorm
    from lingua_amd.swiglu import fuse_feed_forward
    with torch.device("cuda"):
        m = Llama(**CFG).to(torch.bfloat16)
    m.init_weights(0.04, seed=3)
    old = (float8.config.save_fp8_input, float8.config.use_custom_ops)
    if kind != "bf16":
        m = convert_linears_to_fp8(m, "rowwise", r"layers\.[0-9]+\.")
    if kind == "fp8-fused-lean":
        m = fuse_rmsnorm(fuse_feed_forward(m))
        float8.config.save_fp8_input = True
    if kind == "fp8-custom-ops":
        float8.config.use_custom_ops = True
    try:
        master = [p.detach().float().clone() for p in m.parameters()]      # fp32 master weights, bf16 model copies
        opt = torch.optim.AdamW(master, lr=2e-3, weight_decay=0.0)
        g = torch.Generator().manual_seed(4)
        tokens = torch.randint(0, CFG["vocab"], (8, 128), generator=g).cuda()
        labels = torch.roll(tokens, -1, dims=1)
        losses = []
        for _ in range(STEPS):
            loss = m(tokens, labels)
            for p in m.parameters():
                p.grad = None
            loss.backward()
            for p, w in zip(m.parameters(), master):
                w.grad = p.grad.float()
            opt.step()
            with torch.no_grad():
                for p, w in zip(m.parameters(), master):
                    p.copy_(w)                                             # in place: same storage, new version
            losses.append(float(loss.detach()))
    finally:
        float8.config.save_fp8_input, float8.config.use_custom_ops = old
    return losses


def test_every_variant_learns_the_batch_like_the_bf16_model():
    ref = _train("bf16")
    assert ref[-1] < 0.5 * ref[0], ref            # the task is learnable in this many steps
    for kind in ("fp8", "fp8-fused-lean", "fp8-custom-ops"):
        got = _train(kind)
        assert all(torch.isfinite(torch.tensor(got))), (kind, got)
        assert abs(got[0] - ref[0]) < 0.02 * ref[0], (kind, got[0], ref[0])
        assert got[-1] < 0.5 * got[0], (kind, got)
        assert abs(got[-1] - ref[-1]) < 0.15 * ref[-1] + 0.05, (kind, got[-1], ref[-1])


@pytest.mark.parametrize("fused", [False, True])
def test_activation_checkpointing_reproduces_the_plain_backward(fused):
    """Every block under torch.utils.checkpoint (forward run again inside backward, interleaved with the
    backward of the block after it): the quantisation memo must not hand a stale copy to the recomputed pass.
    The kernels are deterministic, so loss and every gradient are bit-identical to the run without it."""
    from torch.utils.checkpoint import checkpoint
    from lingua_amd import convert_linears_to_fp8
    from bench_workloads import Llama, rope_tables
    from lingua_amd.norm import fuse_rmsnorm
    from lingua_amd.swiglu import fuse_feed_forward
    with torch.device("cuda"):
        m = Llama(**CFG).to(torch.bfloat16)
    m.init_weights(0.04, seed=5)
    m = convert_linears_to_fp8(m, "rowwise", r"layers\.[0-9]+\.")
    if fused:
        m = fuse_rmsnorm(fuse_feed_forward(m))
    g = torch.Generator().manual_seed(6)
    tokens = torch.randint(0, CFG["vocab"], (4, 96), generator=g).cuda()
    labels = torch.roll(tokens, -1, dims=1)

    def run(with_ac):
        for p in m.parameters():
            p.grad = None
        cos, sin = rope_tables(m.head_dim, tokens.shape[1], m.rope_theta, tokens.device)
        h = m.tok_embeddings(tokens)
        for layer in m.layers:
            h = checkpoint(layer, h, cos, sin, use_reentrant=False) if with_ac else layer(h, cos, sin)
        logits = m.output(m.norm(h))
        loss = torch.nn.functional.cross_entropy(logits.flatten(0, 1).float(), labels.flatten())
        loss.backward()
        return float(loss.detach()), [p.grad.clone() for p in m.parameters()]

    loss_plain, grads_plain = run(False)
    loss_ac, grads_ac = run(True)
    assert loss_ac == loss_plain
    for (name, _), a, b in zip(m.named_parameters(), grads_ac, grads_plain):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), name
