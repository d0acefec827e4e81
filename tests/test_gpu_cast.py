"""GPU parity of the cast kernels against the CPU oracle: e4m3 bytes, fp32
scales and bf16 amaxes must be bit-identical (NaN codes compare equal
irrespective of sign, see golden_util.fp8_equal_mod_nan_sign)."""
import pytest
import torch

import oracle
from conftest import seeded_bf16
from golden_util import bits_equal, fp8_equal_mod_nan_sign, load_golden

pytestmark = pytest.mark.gpu


def _lib_handle():
    from lingua_amd import _lib
    return _lib.load()


def dev(t):
    return t.to("cuda")


def check_rowwise(x, with_col=False):
    from lingua_amd import ops
    col = torch.full((x.shape[1],), 7e29, dtype=torch.float32, device="cuda") if with_col else None   # stale contents
    q, s, a = ops.cast_rowwise(dev(x), col_amax=col)
    qo, so, ao = oracle.cast_rowwise(x)
    assert torch.equal(q.cpu().view(torch.uint8), qo), "bytes differ"
    assert bits_equal(s.cpu().reshape(-1), so), "scales differ"
    assert bits_equal(a.cpu().reshape(-1), ao), "amax differ"
    if with_col:
        assert bits_equal(col.cpu(), oracle.col_amax(x).float()), "column amax differ"
    return q, s


def test_golden_vectors():
    from lingua_amd import ops
    g = load_golden()
    for name, t in (("x", g["x"]), ("w", g["w"]), ("g", g["go"])):
        q, s, a = ops.cast_rowwise(dev(t))
        assert torch.equal(q.cpu().view(torch.uint8), g["q_" + name]), name
        assert bits_equal(s.cpu().reshape(-1), g["s_" + name]), name
    assert bits_equal(ops.cast_rowwise(dev(g["x"]))[2].cpu().reshape(-1), g["amax_x"])
    w = dev(g["w"])
    _, _, amax_w = ops.cast_rowwise(w, want_q=False)
    qwt, swt = ops.cast_tensorwise(w, ops.amax_reduce(amax_w), transpose=True)
    assert torch.equal(qwt.cpu().view(torch.uint8), g["q_wt"])
    assert bits_equal(swt.cpu().reshape(-1).expand(g["s_wt"].shape).contiguous(), g["s_wt"])
    for name, t in (("gt", g["go"]), ("xt", g["x"])):
        td = dev(t)
        q, s = ops.cast_colwise_transposed(td, ops.col_amax(td))
        assert torch.equal(q.cpu().view(torch.uint8), g["q_" + name]), name
        assert bits_equal(s.cpu().reshape(-1), g["s_" + name]), name
    x = dev(g["x"])
    q, s = ops.cast_tensorwise(x, ops.amax_reduce(ops.cast_rowwise(x, want_q=False)[2]))
    assert torch.equal(q.cpu().view(torch.uint8), g["q_x_tw"]) and bits_equal(s.cpu().reshape(-1), g["s_x_tw"])


@pytest.mark.parametrize("shape", [(1, 8), (3, 16), (7, 520), (5, 4096), (300, 2048), (33, 11008), (9, 12288),
                                   (1027, 1024), (3, 16384), (2, 40000)])
@pytest.mark.parametrize("with_col", [False, True])
def test_rowwise_shapes(shape, with_col):
    x = seeded_bf16(shape, seed=shape[0] * 131 + shape[1])
    x[0, 0] = 0.0
    if shape[0] > 2:
        x[2] = 0.0
    check_rowwise(x, with_col)


def test_rowwise_config1_inputs():
    check_rowwise(seeded_bf16((4096, 2048), 1.0, seed=0), with_col=True)
    check_rowwise(seeded_bf16((2048, 2048), 0.02, seed=1))


def test_rowwise_strided_input_and_col_amax_overwritten():
    from lingua_amd import ops
    big = seeded_bf16((64, 1536), seed=9)
    x = big[:, 256:256 + 1024]              # row stride 1536, offset 512 bytes
    xd = dev(big)[:, 256:256 + 1024]
    col = torch.full((1024,), 1e30, dtype=torch.float32, device="cuda")     # stale contents must not survive
    q, s, a = ops.cast_rowwise(xd, col_amax=col)
    qo, so, ao = oracle.cast_rowwise(x.contiguous())
    assert torch.equal(q.cpu().view(torch.uint8), qo) and bits_equal(s.cpu().reshape(-1), so)
    assert bits_equal(col.cpu(), oracle.col_amax(x.contiguous()).float())
    # the stand-alone column amax and the two-pass kernel for very long rows overwrite as well
    lib = _lib_handle()
    col2 = torch.full((1024,), 1e30, dtype=torch.float32, device="cuda")
    assert lib.l8_col_amax(xd.data_ptr(), 64, 1024, 1536, col2.data_ptr(), torch.cuda.current_stream().cuda_stream) == 0
    assert bits_equal(col2.cpu(), oracle.col_amax(x.contiguous()).float())
    wide = seeded_bf16((3, 40960), seed=10)
    col3 = torch.full((40960,), 1e30, dtype=torch.float32, device="cuda")
    q3, s3, _ = ops.cast_rowwise(dev(wide), col_amax=col3)
    assert torch.equal(q3.cpu().view(torch.uint8), oracle.cast_rowwise(wide)[0])
    assert bits_equal(col3.cpu(), oracle.col_amax(wide).float())


def test_rowwise_nonfinite_rows():
    from lingua_amd import ops
    x = seeded_bf16((6, 1024), seed=4)
    x[1, 3] = float("inf")
    x[2, 5] = float("nan")
    x[3, 7] = float("-inf")
    x[3, 9] = float("nan")
    q, s, a = ops.cast_rowwise(dev(x))
    qo, so, ao = oracle.cast_rowwise(x)
    assert fp8_equal_mod_nan_sign(q, qo)
    s, a = s.cpu().reshape(-1), a.cpu().reshape(-1)
    assert torch.equal(s.isnan(), so.isnan()) and torch.equal(s.isinf(), so.isinf())
    fin = so.isfinite()
    assert bits_equal(s[fin], so[fin])
    assert torch.equal(a.isnan(), ao.isnan()) and bits_equal(a[~ao.isnan()], ao[~ao.isnan()])


@pytest.mark.parametrize("amax", [448.0, 1.0, 0.0123, 3.3895e38, 1e-30, 240.0, 5.5e-13, 7.0])
def test_every_bf16_pattern_through_the_hardware_converter(amax):
    # one row per 4096 patterns; each row's amax is forced to `amax`, larger magnitudes and NaNs are zeroed
    bits = torch.arange(0, 65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(torch.bfloat16).clone().reshape(16, 4096)
    a = torch.tensor(amax).to(torch.bfloat16)
    bad = ~(x.float().abs() <= a.float())
    x[bad] = 0.0
    x[:, 0] = a
    check_rowwise(x)
    # same patterns as one long row (two-pass kernel) and through the transposed kernels
    from lingua_amd import ops
    long_row = x.reshape(1, -1)
    check_rowwise(long_row)
    xd = dev(x)
    qt, st = ops.cast_colwise_transposed(xd, ops.col_amax(xd))
    qo, so = oracle.cast_colwise_transposed(x)
    assert torch.equal(qt.cpu().view(torch.uint8), qo) and bits_equal(st.cpu().reshape(-1), so)
    qw, sw = ops.cast_tensorwise(xd, dev(a.reshape(1, 1)))
    qwo, swo = oracle.cast_tensorwise(x, a)
    assert torch.equal(qw.cpu().view(torch.uint8), qwo) and bits_equal(sw.cpu().reshape(-1), swo)


@pytest.mark.parametrize("shape", [(1, 8), (4, 8), (128, 64), (129, 72), (100, 200), (257, 1000), (2048, 512),
                                   (50, 11008), (1030, 136)])
def test_transposed_kernels_shapes(shape):
    from lingua_amd import ops
    x = seeded_bf16(shape, seed=shape[0] * 7 + shape[1])
    x[0, 0] = 0.0
    if shape[1] > 16:
        x[:, 11] = 0.0  # an all-zero column: scale floor
    xd = dev(x)
    ca = ops.col_amax(xd)
    assert bits_equal(ca.cpu(), oracle.col_amax(x).float())
    q, s = ops.cast_colwise_transposed(xd, ca)
    qo, so = oracle.cast_colwise_transposed(x)
    R = shape[0]
    assert q.shape[1] % 16 == 0 and q.shape[1] - R < 16
    assert torch.equal(q.cpu().view(torch.uint8)[:, :R], qo) and bits_equal(s.cpu().reshape(-1), so)
    assert (q.cpu().view(torch.uint8)[:, R:] == 0).all()      # reduction padding is e4m3 zero
    amax = ops.amax_reduce(ops.cast_rowwise(xd, want_q=False)[2])
    assert bits_equal(amax.cpu().reshape(()), oracle.amax_of_amaxes(oracle.row_amax(x)))
    for tr in (False, True):
        q, s = ops.cast_tensorwise(xd, amax, transpose=tr)
        qo, so = oracle.cast_tensorwise(x, transpose=tr)
        assert torch.equal(q.cpu().view(torch.uint8), qo), tr
        assert bits_equal(s.cpu().reshape(-1), so), tr


def test_colwise_nonfinite_columns():
    from lingua_amd import ops
    x = seeded_bf16((40, 64), seed=6)
    x[3, 5] = float("inf")
    x[7, 9] = float("nan")
    xd = dev(x)
    q, s = ops.cast_colwise_transposed(xd, ops.col_amax(xd))
    qo, so = oracle.cast_colwise_transposed(x)
    assert fp8_equal_mod_nan_sign(q[:, :40], qo)
    s = s.cpu().reshape(-1)
    assert s[5].isinf() and s[9].isnan()
    fin = so.isfinite()
    assert bits_equal(s[fin], so[fin])


@pytest.mark.parametrize("bad", [float("inf"), float("nan")])
@pytest.mark.parametrize("amax_dtype", [torch.bfloat16, torch.float32])
def test_transposed_casts_with_a_nonfinite_amax_over_several_tiles(bad, amax_dtype):
    """The transposed kernels redo a column (or, tensor-wise, everything) whose amax is not finite with the
    integer conversion: ragged shape, more than one tile in both directions, both halves of a tile's rows."""
    from lingua_amd import ops
    x = seeded_bf16((300, 136), seed=11)
    x[1, 3] = bad
    x[140, 70] = bad
    x[299, 135] = bad
    xd = dev(x)
    amax = torch.tensor([[bad]], dtype=amax_dtype)
    for tr in (False, True):
        q, s = ops.cast_tensorwise(xd, dev(amax), transpose=tr)
        qo, so = oracle.cast_tensorwise(x, amax, transpose=tr)
        assert fp8_equal_mod_nan_sign(q.cpu().view(torch.uint8), qo), tr
        s = s.cpu().reshape(-1)
        assert torch.equal(s.isnan(), so.isnan()) and torch.equal(s.isinf(), so.isinf()), tr
    if amax_dtype == torch.float32:
        q, s = ops.cast_colwise_transposed(xd, ops.col_amax(xd))
        qo, so = oracle.cast_colwise_transposed(x)
        assert fp8_equal_mod_nan_sign(q[:, :300].cpu().view(torch.uint8), qo)
        s = s.cpu().reshape(-1)
        fin = so.isfinite()
        assert not fin[3] and not fin[70] and not fin[135] and int(fin.sum()) == 133
        assert bits_equal(s[fin], so[fin])


@pytest.mark.parametrize("ldq_pad", [0, 7])
def test_transposed_casts_with_ragged_edges_on_the_large_tile(ldq_pad):
    """Tensors with at least four 128 x 128 tiles per compute unit take the 128 x 128 tile (smaller ones a 64 x 128
    tile, which the random-shape sweep covers): rows and columns that are not multiples of the tile, a padded input
    row stride, an output row stride that rules out 16-byte stores, and one column with a non-finite amax."""
    from lingua_amd import _lib
    lib = _lib.load()
    R, C, ldx = 4100, 4104, 4112
    g = torch.Generator().manual_seed(21)
    xb = torch.randn(R, ldx, generator=g).to(torch.bfloat16)
    xb[:, C:] = 3.0e38                      # padding columns must not be read
    xb[17, 130] = float("inf")
    x = xb.cuda()
    xc = xb[:, :C].contiguous()
    ldq = (R + 15) // 16 * 16 + ldq_pad
    st = torch.cuda.current_stream().cuda_stream
    col = torch.zeros(C, dtype=torch.float32, device="cuda")
    _lib.check(lib.l8_col_amax(x.data_ptr(), R, C, ldx, col.data_ptr(), st), "l8_col_amax")
    q = torch.full((C, ldq), 0x55, dtype=torch.uint8, device="cuda")
    s = torch.empty(C, dtype=torch.float32, device="cuda")
    _lib.check(lib.l8_cast_colwise_transposed(x.data_ptr(), R, C, ldx, col.data_ptr(), q.data_ptr(), ldq, s.data_ptr(), st),
               "l8_cast_colwise_transposed")
    wq, ws = oracle.cast_colwise_transposed(xc)
    assert fp8_equal_mod_nan_sign(q.cpu()[:, :R], wq)
    assert (q.cpu()[:, R:] == 0x55).all()
    fin = ws.isfinite()
    assert int((~fin).sum()) == 1 and not fin[130] and bits_equal(s.cpu()[fin], ws[fin])
    amax = oracle.amax_of_amaxes(oracle.row_amax(xc[:, :128]))      # a finite amax that does not bound the tensor
    q = torch.full((C, ldq), 0x55, dtype=torch.uint8, device="cuda")
    s1 = torch.empty(1, dtype=torch.float32, device="cuda")
    xfin = xb.clone()
    xfin[17, 130] = 1.0
    xfin[:, :C] = xfin[:, :C].clamp(-float(amax.float()), float(amax.float()))
    _lib.check(lib.l8_cast_tensorwise(xfin.cuda().data_ptr(), R, C, ldx, amax.cuda().data_ptr(), 0, 1, q.data_ptr(), ldq,
                                      s1.data_ptr(), st), "l8_cast_tensorwise")
    wq, ws = oracle.cast_tensorwise(xfin[:, :C].contiguous(), amax, transpose=True)
    assert torch.equal(q.cpu()[:, :R], wq) and (q.cpu()[:, R:] == 0x55).all() and bits_equal(s1.cpu(), ws.reshape(-1))


def test_transposed_casts_with_ragged_edges_on_the_tall_tile():
    """Tensors of at least 16384 rows and 8192 columns take a 128 x 256 tile: same edge cases as for the other tiles,
    the whole output against the C oracle."""
    from lingua_amd import _lib
    lib = _lib.load()
    R, C, ldx = 16390, 8200, 8208
    g = torch.Generator().manual_seed(22)
    xb = torch.randn(R, ldx, generator=g).to(torch.bfloat16)
    xb[:, C:] = 3.0e38                      # padding columns must not be read
    xb[16389, 8199] = float("nan")
    x = xb.cuda()
    xc = xb[:, :C].contiguous()
    st = torch.cuda.current_stream().cuda_stream
    col = torch.zeros(C, dtype=torch.float32, device="cuda")
    _lib.check(lib.l8_col_amax(x.data_ptr(), R, C, ldx, col.data_ptr(), st), "l8_col_amax")
    for ldq in (16400, 16391):              # 16-byte stores, byte stores
        q = torch.full((C, ldq), 0x55, dtype=torch.uint8, device="cuda")
        s = torch.empty(C, dtype=torch.float32, device="cuda")
        _lib.check(lib.l8_cast_colwise_transposed(x.data_ptr(), R, C, ldx, col.data_ptr(), q.data_ptr(), ldq, s.data_ptr(), st),
                   "l8_cast_colwise_transposed")
        wq, ws = oracle.cast_colwise_transposed(xc)
        assert fp8_equal_mod_nan_sign(q[:, :R].cpu(), wq), ldq
        assert bool((q[:, R:] == 0x55).all()), ldq
        fin = ws.isfinite()
        assert int((~fin).sum()) == 1 and not fin[8199] and bits_equal(s.cpu()[fin], ws[fin]), ldq


from bench_workloads import outlier_stress_input  # noqa: E402


def test_outlier_stress_full_size_rowwise_tensorwise_colwise():
    from lingua_amd import ops
    x, ch, zr = outlier_stress_input()
    xd = dev(x)
    col = torch.zeros(x.shape[1], dtype=torch.float32, device="cuda")
    q, s, a = ops.cast_rowwise(xd, col_amax=col)
    qo, so, ao = oracle.cast_rowwise(x)
    assert torch.equal(q.cpu().view(torch.uint8), qo)
    assert bits_equal(s.cpu().reshape(-1), so) and bits_equal(a.cpu().reshape(-1), ao)
    assert (s.cpu().reshape(-1)[zr].view(torch.int32) == 0x2720D7C5).all()
    assert (q.cpu().view(torch.uint8)[zr] == 0).all()
    assert bits_equal(col.cpu(), oracle.col_amax(x).float())
    amax = ops.amax_reduce(a)
    qt, st = ops.cast_tensorwise(xd, amax)
    qto, sto = oracle.cast_tensorwise(x)
    assert torch.equal(qt.cpu().view(torch.uint8), qto) and bits_equal(st.cpu().reshape(-1), sto)
    qc, sc = ops.cast_colwise_transposed(xd, col)
    qco, sco = oracle.cast_colwise_transposed(x)
    assert torch.equal(qc.cpu().view(torch.uint8), qco) and bits_equal(sc.cpu().reshape(-1), sco)
    # row-wise scaling keeps far more of the signal than one scale for the whole tensor
    xf = x.float()
    deq_r = q.cpu().float() * s.cpu()
    deq_t = qt.cpu().float() * st.cpu()
    err_r = (deq_r - xf).norm() / xf.norm()
    err_t = (deq_t - xf).norm() / xf.norm()
    assert err_r < err_t


def test_ffn_hidden_shape_properties_full_size():
    # [16384, 11008]: too large for a full oracle pass to be cheap; checked through properties and a row sample
    from lingua_amd import ops
    g = torch.Generator(device="cuda").manual_seed(0)
    h = torch.randn(16384, 11008, generator=g, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    col = torch.zeros(11008, dtype=torch.float32, device="cuda")
    q, s, a = ops.cast_rowwise(h, col_amax=col)
    qb = q.view(torch.uint8)
    assert ((qb & 0x7F).amax(dim=1) == 0x7E).all()          # every row reaches +-448
    assert torch.equal(a.reshape(-1), h.abs().amax(dim=1))
    assert torch.equal(col, h.abs().amax(dim=0).float())
    rows = torch.arange(0, 16384, 257)
    qo, so, _ = oracle.cast_rowwise(h[rows.cuda()].cpu())
    assert torch.equal(qb[rows.cuda()].cpu(), qo) and bits_equal(s.reshape(-1)[rows.cuda()].cpu(), so)
    # transposed cast == row-wise cast of the transpose, both on the GPU
    qt, st = ops.cast_colwise_transposed(h, col)
    ht = h.t().contiguous()
    q2, s2, _ = ops.cast_rowwise(ht)
    assert torch.equal(qt.view(torch.uint8), q2.view(torch.uint8)) and torch.equal(st, s2)


def test_every_finite_amax_lands_on_448_in_the_hardware_converter():
    """One row (and one column) per finite positive bf16 amax, bit patterns 0x0001 .. 0x7F7F: element 0 is the amax,
    so `amax * (1 / scale)` -- which may exceed 448 by an ulp or two -- goes through the hardware converter for
    every amax there is, in the row-wise kernel and in the transposed one (lingua/float8.py:43-47); the other
    elements are random magnitudes below it."""
    from lingua_amd import ops
    n = 0x7F7F
    g = torch.Generator().manual_seed(77)
    amax_bits = torch.arange(1, n + 1, dtype=torch.int32)
    C = 16
    frac = torch.rand(n, C, generator=g)
    mag = (frac * (amax_bits.reshape(n, 1) + 1).float()).to(torch.int32).clamp_(max=amax_bits.reshape(n, 1))
    sign = torch.randint(0, 2, (n, C), generator=g, dtype=torch.int32) << 15
    bits = mag | sign
    bits[:, 0] = amax_bits
    x = bits.to(torch.int16).view(torch.bfloat16)
    rows = torch.zeros(n + 1, C, dtype=torch.bfloat16)   # + one zero row: a multiple of 8 columns once transposed
    rows[:n] = x
    q, s = check_rowwise(rows)
    above_floor = rows[:n, 0].float() >= 1e-12                       # smaller amaxes are lifted to the floor of the scale
    assert bool((q.cpu().view(torch.uint8)[:n, 0][above_floor] == 0x7E).all())   # every other amax quantises to +448
    # the same values with one amax per column, through the transposed kernel
    xt = rows.t().contiguous()                                       # [16, 32640]
    xd = dev(xt)
    col = ops.col_amax(xd)
    assert bits_equal(col.cpu(), oracle.col_amax(xt).float())
    qt, st = ops.cast_colwise_transposed(xd, col)
    qo, so = oracle.cast_colwise_transposed(xt)
    assert torch.equal(qt.cpu().view(torch.uint8), qo) and bits_equal(st.cpu().reshape(-1), so)
    assert torch.equal(qt.cpu().view(torch.uint8), q.cpu().view(torch.uint8))  # same bytes either way


def test_pytorchs_gpu_division_by_a_scalar_is_the_product_with_the_inverse():
    """What `torch.clamp(amax_t.float(), min=EPS) / FP8_MAX` (lingua/float8.py:44) gives on this GPU, for every
    non-negative bf16 amax: PyTorch's GPU kernel multiplies by fp32(1/448), its CPU kernel divides, and the two differ
    in the last bit for a good third of the amaxes.  This pins the oracle's "times_inverse" rule against PyTorch's own
    kernel; the default rule is pinned against the CPU kernel in tests/test_oracle_cast.py."""
    bits = torch.arange(0, 0x7F81, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    on_gpu = (torch.clamp(bits.cuda().float(), min=1e-12) / 448.0).cpu()
    on_cpu = torch.clamp(bits.float(), min=1e-12) / 448.0
    assert bits_equal(oracle.scale_from_amax(bits), on_cpu)
    with oracle.scale_rule("times_inverse"):
        assert bits_equal(oracle.scale_from_amax(bits), on_gpu)
    differ = (on_gpu.view(torch.int32) != on_cpu.view(torch.int32)).float().mean().item()
    assert 0.2 < differ < 0.6


@pytest.mark.parametrize("shape", [(4096, 2048), (777, 1000), (64, 11008), (3, 8)])
def test_casts_under_the_gpu_division_rule_equal_pytorchs_own_gpu_ops(shape, gpu_division_rule):
    """With `lingua_amd.set_scale_rule("times_inverse")` every layout's bytes and scales equal, bit for bit, what the
    reference's op chain (oracle.recipe_torch issues it op for op) gives when PyTorch runs it on this GPU -- and the
    oracle under the same rule."""
    from oracle import recipe_torch as rt
    from lingua_amd import ops
    x = seeded_bf16(shape, 1.0, seed=shape[0] + shape[1])
    x[0, 0] = 0
    if shape[0] > 2:
        x[1] = 0                      # a zero row: the floor of the clamp under this rule
    xd = x.cuda()
    # row-wise
    q, s, a = ops.cast_rowwise(xd)
    q_t, s_t = rt.scale(xd, rt.row_amax(xd))
    assert bits_equal(q.view(torch.uint8), q_t.view(torch.uint8)) and bits_equal(s.reshape(-1), s_t.reshape(-1))
    q_o, s_o, _ = oracle.cast_rowwise(x)
    assert torch.equal(q.cpu().view(torch.uint8), q_o) and bits_equal(s.cpu().reshape(-1), s_o)
    # an amax of the caller's, fp32
    amax32 = rt.row_amax(xd).float() * 1.5
    q, s = ops.cast_rowwise_given_amax(xd, amax32)
    q_t, s_t = rt.scale(xd, amax32)
    assert bits_equal(q.view(torch.uint8), q_t.view(torch.uint8)) and bits_equal(s.reshape(-1), s_t.reshape(-1))
    # column-wise, transposed (the wgrad operands)
    col = torch.zeros(shape[1], dtype=torch.float32, device="cuda")
    ops.cast_rowwise(xd, col_amax=col)
    q, s = ops.cast_colwise_transposed(xd, col)
    xt = xd.t().contiguous()
    q_t, s_t = rt.scale(xt, rt.row_amax(xt))
    assert bits_equal(q[:, :shape[0]].contiguous().view(torch.uint8), q_t.view(torch.uint8)) and bits_equal(s.reshape(-1), s_t.reshape(-1))
    # one scale for the tensor, both layouts
    amax = xd.abs().amax().reshape(1, 1)
    for transpose in (False, True):
        q, s = ops.cast_tensorwise(xd, amax, transpose=transpose)
        q_t, s_t = rt.scale(xt if transpose else xd, amax)
        cols = shape[0] if transpose else shape[1]
        assert bits_equal(q[:, :cols].contiguous().view(torch.uint8), q_t.view(torch.uint8)) and bits_equal(s.reshape(-1), s_t.reshape(-1))
