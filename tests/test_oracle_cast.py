"""Pins the oracle's scalar routines (CPU only).

Each check compares the C restatement with something that does not share its
code: PyTorch's own CPU cast, a brute-force nearest-value search over the 256
decoded codes, numpy float32 division, closed-form bit patterns.
"""
import numpy as np
import pytest
import torch

import oracle


def _all_bf16_as_f32():
    bits = torch.arange(0, 65536, dtype=torch.int32)
    return (bits << 16).view(torch.float32)


def test_decode_table_matches_torch():
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float()
    mine = oracle.e4m3fn_decode_table()
    both_nan = ref.isnan() & mine.isnan()
    assert torch.equal(ref.isnan(), mine.isnan())
    assert torch.equal(ref[~both_nan].view(torch.int32), mine[~both_nan].view(torch.int32))  # bit-equal incl. -0
    assert ref.isnan().sum() == 2  # 0x7F and 0xFF only


def test_cast_vs_torch_library_dense_sample():
    # every bf16 pattern (upper 16 bits) x 64 random lower halves + the all-zero / all-one lower halves
    g = torch.Generator().manual_seed(1)
    hi = torch.arange(0, 65536, dtype=torch.int64) << 16
    lows = torch.cat([torch.tensor([0, 0xFFFF, 0x8000, 0x7FFF, 0x8001]), torch.randint(0, 65536, (64,), generator=g)])
    w = (hi[:, None] | lows[None, :]).reshape(-1)
    w32 = torch.where(w >= 2**31, w - 2**32, w).to(torch.int32)
    x = w32.view(torch.float32)
    ref = x.to(torch.float8_e4m3fn).view(torch.uint8)
    mine = oracle.e4m3fn_from_f32(x)
    nan = x.isnan()
    assert torch.equal(ref[~nan], mine[~nan])
    # NaN inputs give the NaN code; the sign is kept
    assert torch.equal(mine[nan] & 0x7F, torch.full_like(mine[nan], 0x7F))
    assert torch.equal(ref[nan], mine[nan])


def test_cast_is_round_to_nearest_even_by_brute_force():
    # independent definition: nearest decoded value, ties to the even code, >=480 -> NaN code
    dec = oracle.e4m3fn_decode_table().double()
    finite_codes = [c for c in range(0, 0x7F)]  # non-negative finite codes, increasing
    vals = dec[finite_codes]
    g = torch.Generator().manual_seed(2)
    xs = torch.cat([
        torch.rand(20000, generator=g, dtype=torch.float64) * 500.0,
        torch.rand(20000, generator=g, dtype=torch.float64) * 0.05,
        (vals[:-1] + vals[1:]) / 2,            # every exact midpoint
        vals,                                    # every exact value
        torch.tensor([464.0, 464.00003, 479.99997, 480.0, 2.0 ** -10, 2.0 ** -10 * 1.0000001, 2.0 ** -11]),
    ]).float()
    got = oracle.e4m3fn_from_f32(xs)
    for x, c in zip(xs.double().tolist(), got.tolist()):
        if x >= 480.0:
            assert c == 0x7F
            continue
        d = (vals - x).abs()
        best = d.min()
        cands = [finite_codes[i] for i in torch.nonzero(d == best).flatten().tolist()]
        # beyond 448 the next "value" would be 480 (the NaN code position): 448 < x <= 464 -> 448, above -> NaN code
        if x > 448.0:
            want = 0x7E if x <= 464.0 else 0x7F
        elif len(cands) == 1:
            want = cands[0]
        else:
            want = [c_ for c_ in cands if c_ % 2 == 0][0]
        assert c == want, (x, c, want)
    # sign symmetry
    neg = oracle.e4m3fn_from_f32(-xs)
    assert torch.equal(neg, got | 0x80)


def test_cast_known_answers():
    x = torch.tensor([448., 464., 465., 480., 1e9, float("inf"), 2.0 ** -10, 1.5 * 2.0 ** -10, 2.0 ** -9, 17., 19., -0.0, 0.0,
                      2.0 ** -6, 0.875 * 2.0 ** -6, 1.0, -1.0, 0.9375 * 2.0 ** -6])
    want = torch.tensor([0x7E, 0x7E, 0x7F, 0x7F, 0x7F, 0x7F, 0x00, 0x01, 0x01, 0x58, 0x5A, 0x80, 0x00,
                         0x08, 0x07, 0x38, 0xB8, 0x08], dtype=torch.uint8)
    assert torch.equal(oracle.e4m3fn_from_f32(x), want)


def test_scale_exhaustive_vs_numpy():
    bits = np.arange(0, 0x7F81, dtype=np.uint32)  # every non-negative bf16 up to +inf
    amax_f32 = (bits << 16).view(np.float32)
    with np.errstate(over="ignore"):
        want = np.maximum(amax_f32, np.float32(1e-12)) / np.float32(448.0)
    assert want.dtype == np.float32
    amax = torch.from_numpy(amax_f32.copy()).to(torch.bfloat16)
    got = oracle.scale_from_amax(amax).numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # and against torch's own clamp / div chain
    t = (torch.clamp(amax.float(), min=1e-12) / 448.0).numpy()
    assert np.array_equal(got.view(np.uint32), t.view(np.uint32))


def test_scale_edge_bits():
    z = oracle.scale_from_amax(torch.zeros(1, dtype=torch.bfloat16))
    assert z.view(torch.int32).item() == 0x2720D7C5          # 1e-12f / 448f
    assert np.float32(1e-12).view(np.uint32) == 0x2B8CBCCC
    r = (1.0 / z).view(torch.int32).item()
    assert r == 0x57CBBA10                                     # 4.48e14
    n = oracle.scale_from_amax(torch.tensor([float("nan")], dtype=torch.bfloat16))
    assert n.isnan().all()
    i = oracle.scale_from_amax(torch.tensor([float("inf")], dtype=torch.bfloat16))
    assert i.isinf().all()


def test_amax_times_recip_lands_on_448_for_every_amax():
    # for every finite positive bf16 amax >= the floor, amax * (1/scale) rounds to the code of 448
    bits = torch.arange(1, 0x7F80, dtype=torch.int32)
    amax = (bits << 16).view(torch.float32)
    amax = amax[amax >= 1e-12]
    s = oracle.scale_from_amax(amax.to(torch.bfloat16))
    p = amax * (1.0 / s)
    codes = oracle.e4m3fn_from_f32(p)
    assert (codes == 0x7E).all()
    assert float(p.max()) < 464.0 and float(p.min()) > 432.0


def test_row_and_col_amax_bruteforce_and_nan():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(37, 40, generator=g).to(torch.bfloat16)
    assert torch.equal(oracle.row_amax(x), x.abs().amax(dim=1))
    assert torch.equal(oracle.col_amax(x), x.abs().amax(dim=0))
    x[5, 7] = float("nan")
    x[9, 3] = float("-inf")
    ra, ca = oracle.row_amax(x), oracle.col_amax(x)
    assert ra[5].isnan() and ca[7].isnan() and ra[9].isinf() and ca[3].isinf()
    assert torch.equal(ra.isnan(), x.abs().amax(dim=1).isnan())
    tot = oracle.amax_of_amaxes(ra)
    assert tot.isnan()
    y = x.clone(); y[5, 7] = 0
    assert oracle.amax_of_amaxes(oracle.row_amax(y)).isinf()


def test_scale_under_the_gpu_division_rule_exhaustive_vs_numpy():
    """ATen's GPU kernel divides a tensor by a Python scalar by multiplying with fp32(1/scalar); under
    oracle.scale_rule("times_inverse") the oracle does the same.  Every non-negative bf16 amax against numpy float32
    arithmetic; the rule must change the last bit of a good part of the scales (else it would pin nothing) and must
    leave amax * (1/scale) on the code of 448 all the same.  (That PyTorch's GPU kernel really computes this product
    is checked on the GPU, tests/test_gpu_cast.py.)"""
    bits = np.arange(0, 0x7F81, dtype=np.uint32)
    amax_f32 = (bits << 16).view(np.float32)
    inv = np.float32(1.0) / np.float32(448.0)
    with np.errstate(over="ignore"):
        want = np.maximum(amax_f32, np.float32(1e-12)) * inv
        quotient = np.maximum(amax_f32, np.float32(1e-12)) / np.float32(448.0)
    amax = torch.from_numpy(amax_f32.copy()).to(torch.bfloat16)
    with oracle.scale_rule("times_inverse"):
        got = oracle.scale_from_amax(amax).numpy()
        from oracle import recipe_torch as rt
        _, chain = rt.scale(torch.zeros(amax.numel(), 1, dtype=torch.bfloat16), amax.reshape(-1, 1))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.array_equal(chain.numpy().reshape(-1).view(np.uint32), want.view(np.uint32))
    differ = (got.view(np.uint32) != quotient.view(np.uint32)).mean()
    assert 0.2 < differ < 0.6
    assert np.abs(got.view(np.int32).astype(np.int64) - quotient.view(np.int32).astype(np.int64)).max() == 1
    # back under the default rule the quotient is what comes out
    assert np.array_equal(oracle.scale_from_amax(amax).numpy().view(np.uint32), quotient.view(np.uint32))
    fin = torch.from_numpy(amax_f32[(amax_f32 >= 1e-12) & np.isfinite(amax_f32)].copy())
    with oracle.scale_rule("times_inverse"):
        s = oracle.scale_from_amax(fin.to(torch.bfloat16))
    p = fin * (1.0 / s)
    assert (oracle.e4m3fn_from_f32(p) == 0x7E).all() and float(p.max()) < 464.0 and float(p.min()) > 432.0
