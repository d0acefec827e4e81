"""Minimal stand-ins for the call sites of the fp8 linear path, with the module
names of the reference so that the default filter ``layers\\.[0-9]+\\.`` selects
the same layers (wq/wk/wv/wo/w1/w2/w3 in every block, not ``output`` /
``tok_embeddings``; lingua/distributed.py:69-70).

They exist so that tests and benchmarks can drive ``convert_linears_to_fp8``
the way lingua's ``parallelize_model`` does (lingua/distributed.py:403-406);
everything that is not a linear runs on plain PyTorch ops.  Also here: the
seeded synthetic inputs that tests and benchmark share.  Not part of the
product package.

  * ``FeedForward``      SwiGLU MLP, lingua/transformer.py:430-471
  * ``Attention``        lingua/transformer.py:306-410 (causal sdpa path only)
  * ``TransformerBlock`` lingua/transformer.py:497-543
  * ``Llama``            tok_embeddings / layers / norm / output as in
                         apps/main/transformer.py:74-119, cross-entropy loss
"""
import math

import torch
import torch.nn.functional as F
from torch import nn


class RMSNorm(nn.Module):
    def __init__(self, dim: int, eps: float = 1e-5):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        xf = x.float()
        out = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)
        return (out * self.weight.float()).type_as(x)


class FeedForward(nn.Module):
    def __init__(self, dim: int, hidden_dim: int):
        super().__init__()
        self.w1 = nn.Linear(dim, hidden_dim, bias=False)
        self.w3 = nn.Linear(dim, hidden_dim, bias=False)
        self.w2 = nn.Linear(hidden_dim, dim, bias=False)

    def forward(self, x):
        return self.w2(F.silu(self.w1(x)) * self.w3(x))


def rope_tables(head_dim: int, seq_len: int, theta: float, device):
    freqs = 1.0 / (theta ** (torch.arange(0, head_dim, 2, device=device).float() / head_dim))
    ang = torch.outer(torch.arange(seq_len, device=device).float(), freqs)
    return ang.cos(), ang.sin()


def apply_rope(x, cos, sin):
    # x: [B, S, H, D]; rotate pairs (2i, 2i+1)
    xf = x.float().unflatten(-1, (-1, 2))
    a, b = xf[..., 0], xf[..., 1]
    c, s = cos[None, :, None, :], sin[None, :, None, :]
    return torch.stack((a * c - b * s, a * s + b * c), dim=-1).flatten(-2).type_as(x)


class Attention(nn.Module):
    def __init__(self, dim: int, n_heads: int, head_dim: int):
        super().__init__()
        self.n_heads, self.head_dim = n_heads, head_dim
        self.wq = nn.Linear(dim, n_heads * head_dim, bias=False)
        self.wk = nn.Linear(dim, n_heads * head_dim, bias=False)
        self.wv = nn.Linear(dim, n_heads * head_dim, bias=False)
        self.wo = nn.Linear(n_heads * head_dim, dim, bias=False)

    def forward(self, x, cos, sin):
        B, S, _ = x.shape
        q = self.wq(x).view(B, S, self.n_heads, self.head_dim)
        k = self.wk(x).view(B, S, self.n_heads, self.head_dim)
        v = self.wv(x).view(B, S, self.n_heads, self.head_dim)
        q, k = apply_rope(q, cos, sin), apply_rope(k, cos, sin)
        o = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), is_causal=True)
        return self.wo(o.transpose(1, 2).reshape(B, S, self.n_heads * self.head_dim))


class TransformerBlock(nn.Module):
    def __init__(self, dim: int, n_heads: int, head_dim: int, ffn_dim: int, norm_eps: float = 1e-5):
        super().__init__()
        self.attention = Attention(dim, n_heads, head_dim)
        self.feed_forward = FeedForward(dim, ffn_dim)
        self.attention_norm = RMSNorm(dim, norm_eps)
        self.ffn_norm = RMSNorm(dim, norm_eps)

    def forward(self, x, cos, sin):
        h = x + self.attention(self.attention_norm(x), cos, sin)
        return h + self.feed_forward(self.ffn_norm(h))


class Llama(nn.Module):
    def __init__(self, n_layers: int, dim: int, n_heads: int, ffn_dim: int, vocab: int, rope_theta: float = 10000.0):
        super().__init__()
        self.dim, self.head_dim, self.rope_theta = dim, dim // n_heads, rope_theta
        self.tok_embeddings = nn.Embedding(vocab, dim)
        self.layers = nn.ModuleList([TransformerBlock(dim, n_heads, dim // n_heads, ffn_dim) for _ in range(n_layers)])
        self.norm = RMSNorm(dim)
        self.output = nn.Linear(dim, vocab, bias=False)

    @torch.no_grad()
    def init_weights(self, std: float = 0.02, seed: int = 0):
        g = torch.Generator(device=self.tok_embeddings.weight.device).manual_seed(seed)
        for name, p in self.named_parameters():
            if name.endswith("norm.weight"):
                p.fill_(1.0)
            else:
                p.copy_((torch.randn(p.shape, generator=g, device=p.device, dtype=torch.float32) * std).to(p.dtype))

    def forward(self, tokens, labels=None):
        B, S = tokens.shape
        cos, sin = rope_tables(self.head_dim, S, self.rope_theta, tokens.device)
        h = self.tok_embeddings(tokens)
        for layer in self.layers:
            h = layer(h, cos, sin)
        logits = self.output(self.norm(h))
        if labels is None:
            return logits
        return F.cross_entropy(logits.flatten(0, 1).float(), labels.flatten())


def llama_flops_per_token(n_layers: int, dim: int, ffn_dim: int, vocab: int, seq_len: int) -> float:
    """Forward + backward flop per token in the convention of apps/main/transformer.py:46-56:
    6 x (non-embedding parameters) + causal attention."""
    params = n_layers * (4 * dim * dim + 3 * dim * ffn_dim) + dim * vocab
    attn = 3.5 * (4 * n_layers * seq_len * dim // 2)
    return 6.0 * params + attn


LLAMA_1B = dict(n_layers=25, dim=2048, n_heads=16, ffn_dim=8192, vocab=128256)


# ----------------------------------------------------------------------------
# seeded synthetic inputs shared by the tests and the benchmark
# ----------------------------------------------------------------------------

def seeded_bf16(shape, std=1.0, seed=0):
    """fp32 normal on the CPU generator, rounded to bf16 (identical bits for CPU oracle and GPU)."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-300))


def outlier_stress_input(rows=16384, cols=4096, seed=0):
    """Student-t (df=3) activations, 0.1 % of channels x100, 1 % of rows all-zero."""
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(rows, cols, generator=g)
    chi = torch.randn(3, rows, cols, generator=g).pow_(2).sum(0)
    x = z / (chi / 3.0).sqrt_()
    del z, chi
    ch = torch.randperm(cols, generator=g)[: max(1, cols // 1000)]
    x[:, ch] *= 100.0
    zr = torch.randperm(rows, generator=g)[: max(1, rows // 100)]
    x[zr] = 0.0
    return x.to(torch.bfloat16), ch, zr


def outlier_stress_figures(tokens: int = 16384):
    """The 4096 -> 11008 linear on the outlier-stress activations, row-wise against tensor-wise scaling of both
    operands.  Returns the reported figures -- quantisation SNR of x (dB) and rel-L2 of the output against the fp32
    product of the unquantised operands, for either recipe -- and the GPU tensors they were computed from."""
    from lingua_amd import ops
    x, ch, zr = outlier_stress_input(rows=tokens, cols=4096, seed=0)
    w = seeded_bf16((11008, 4096), 0.02, seed=1)
    xd, wd = x.cuda(), w.cuda()
    qx, sx, ax = ops.cast_rowwise(xd)
    qw, sw, aw = ops.cast_rowwise(wd)
    y_row = ops.gemm_nt(qx, qw, sx, sw)
    qxt, sxt = ops.cast_tensorwise(xd, ops.amax_reduce(ax))
    qwt, swt = ops.cast_tensorwise(wd, ops.amax_reduce(aw))
    y_ten = ops.gemm_nt(qxt, qwt, sxt, swt)
    exact = xd.float() @ wd.float().t()

    def snr_db(q, s):
        err = (q.float() * s - xd.float()).double().pow(2).sum()
        return 10.0 * math.log10(float(xd.double().pow(2).sum() / err))

    def err(y):
        return float((y.double() - exact.double()).norm() / exact.double().norm())

    figures = {"tokens": tokens, "snr_x_rowwise_db": round(snr_db(qx, sx), 2), "snr_x_tensorwise_db": round(snr_db(qxt, sxt), 2),
               "rel_l2_y_rowwise": float(f"{err(y_row):.4e}"), "rel_l2_y_tensorwise": float(f"{err(y_ten):.4e}")}
    return figures, dict(x=x, w=w, zero_rows=zr, qx=qx, sx=sx, qw=qw, sw=sw, qxt=qxt, sxt=sxt, qwt=qwt, swt=swt,
                         y_row=y_row, y_ten=y_ten)
