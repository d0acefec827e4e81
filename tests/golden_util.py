import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "recipe_small.npz")


def load_golden():
    z = np.load(GOLDEN, allow_pickle=False)
    out = {}
    for k in z.files:
        a = z[k]
        if a.dtype == np.uint16:
            out[k] = torch.from_numpy(a.astype(np.int16)).view(torch.bfloat16)
        elif a.dtype == np.uint32:
            out[k] = torch.from_numpy(a.astype(np.int32)).view(torch.float32)
        else:
            out[k] = torch.from_numpy(a.copy())
    return out


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Bit-for-bit equality of two tensors of the same dtype (NaN == NaN, -0 != +0)."""
    a, b = a.detach().cpu().contiguous(), b.detach().cpu().contiguous()
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    view = {1: torch.uint8, 2: torch.int16, 4: torch.int32, 8: torch.int64}[a.element_size()]
    return torch.equal(a.view(view), b.view(view))


def fp8_equal_mod_nan_sign(a: torch.Tensor, b: torch.Tensor) -> bool:
    """e4m3 bytes equal, except that the two NaN codes 0x7F / 0xFF compare equal:
    the sign of a NaN produced by inf*0 differs between x86 and the GPU."""
    a = a.detach().cpu().contiguous().view(torch.uint8)
    b = b.detach().cpu().contiguous().view(torch.uint8)
    if a.shape != b.shape:
        return False
    a = torch.where((a & 0x7F) == 0x7F, torch.full_like(a, 0x7F), a)
    b = torch.where((b & 0x7F) == 0x7F, torch.full_like(b, 0x7F), b)
    return torch.equal(a, b)
