"""Writes tests/golden/recipe_small.npz.

The expected values come from PyTorch CPU ops issued in the order of the
reference recipe (oracle/recipe_torch.py); the reference repository itself is
not imported.  Run from the repository root:  python tests/golden/make_golden.py
Arrays are raw bit patterns (uint8 / uint16 / uint32) so the file loads with
numpy.load(allow_pickle=False).
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import recipe_torch as rt  # noqa: E402


def bf16_bits(t):
    return t.contiguous().view(torch.int16).numpy().astype(np.uint16)


def f32_bits(t):
    return t.contiguous().view(torch.int32).numpy().astype(np.uint32)


def fp8_bits(t):
    return t.contiguous().view(torch.uint8).numpy()


def main():
    g = torch.Generator().manual_seed(0)
    M, K, N = 64, 128, 48
    x = torch.randn(M, K, generator=g).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16)
    go = (torch.randn(M, N, generator=g) * 1e-2).to(torch.bfloat16)
    bias = (torch.randn(N, generator=g) * 0.1).to(torch.bfloat16)
    # edge rows: zeros, negative zeros, a bf16 subnormal row, the largest finite bf16, exact ties
    x[3] = 0
    x[4] = -0.0
    x[5] = torch.tensor(1e-40).to(torch.bfloat16)
    x[6, :] = torch.tensor(3.3895e38).to(torch.bfloat16)
    x[6, 1] = 1.0
    x[7, :] = torch.arange(K, dtype=torch.float32).to(torch.bfloat16)
    x[7, 0] = 448.0  # amax 448 -> scale 1 -> products are the integers themselves (17 -> 16, 19 -> 20 ...)
    x[7, 1:] = torch.clamp(x[7, 1:], max=448.0)

    out = {"x": bf16_bits(x), "w": bf16_bits(w), "go": bf16_bits(go), "bias": bf16_bits(bias)}
    qx, sx = rt.scale(x, rt.row_amax(x))
    qw, sw = rt.scale(w, rt.row_amax(w))
    qg, sg = rt.scale(go, rt.row_amax(go))
    b = w.t().contiguous()
    qwt, swt = rt.scale(b, rt.tensor_amax_from_rows(rt.row_amax(w), b.shape[0]))
    gt, xt = go.t().contiguous(), x.t().contiguous()
    qgt, sgt = rt.scale(gt, rt.row_amax(gt))
    qxt, sxt = rt.scale(xt, rt.row_amax(xt))
    qx_tw, sx_tw = rt.scale(x, x.abs().amax().reshape(1, 1))
    for name, q, s in (("x", qx, sx), ("w", qw, sw), ("g", qg, sg), ("wt", qwt, swt), ("gt", qgt, sgt), ("xt", qxt, sxt),
                       ("x_tw", qx_tw, sx_tw)):
        out["q_" + name] = fp8_bits(q)
        out["s_" + name] = f32_bits(s.reshape(-1))
    out["amax_x"] = bf16_bits(rt.row_amax(x).reshape(-1))
    # products: the 3.4e38 row would overflow fp32 once dequantised, so it is replaced for them
    xp = x.clone()
    xp[6] = torch.randn(K, generator=g).to(torch.bfloat16)
    out["x_prod"] = bf16_bits(xp)
    out["y"] = bf16_bits(rt.linear_forward(xp, w, bias))
    out["dx"] = bf16_bits(rt.linear_dgrad(go, w))
    out["dw_fp8"] = bf16_bits(rt.linear_wgrad_fp8(go, xp))
    out["dw_bf16"] = bf16_bits(rt.linear_wgrad_bf16(go, xp))
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "recipe_small.npz"), **out)
    print({k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
