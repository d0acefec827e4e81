"""Seeded sweep over ragged shapes and leading dimensions, called through the C ABI itself (not the Python
wrappers, which always pass dense buffers): every cast kernel bit-exact against the C oracle, the GEMM exact on
integer-valued operands; the bytes between the end of a row and the leading dimension must stay untouched."""
import random

import pytest
import torch

import oracle
from golden_util import bits_equal

pytestmark = pytest.mark.gpu

FILL = 0x5A   # pattern put into every output buffer first; whatever the kernel does not own must keep it


def _lib():
    from lingua_amd import _lib
    return _lib.load(), _lib


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _bf16_rows(rng, R, C, ld, seed):
    """[R, ld] buffer whose first C columns are the operand (normal values, a zero row, an outlier)."""
    g = torch.Generator().manual_seed(seed)
    buf = (torch.randn(R, ld, generator=g) * (10.0 ** rng.uniform(-3, 3))).to(torch.bfloat16)
    if R > 2:
        buf[rng.randrange(R), :C] = 0.0
    buf[rng.randrange(R), rng.randrange(C)] = 3000.0
    return buf


def _shapes(rng, n, max_r, max_c, c_mult):
    out = []
    for _ in range(n):
        R = rng.choice([1, 2, 3, rng.randrange(1, max_r), rng.randrange(1, max_r)])
        C = c_mult * rng.randrange(1, max_c // c_mult + 1)
        ld = C + c_mult * rng.choice([0, 0, 1, 3, 8])
        out.append((R, C, ld))
    return out


def test_cast_rowwise_sweep():
    lib, L = _lib()
    rng = random.Random(1)
    for case, (R, C, ldx) in enumerate(_shapes(rng, 60, 700, 9000, 8)):
        ldq = C + 8 * rng.choice([0, 2, 5])
        xb = _bf16_rows(rng, R, C, ldx, case)
        x = xb.cuda()
        q = torch.full((R, ldq), FILL, dtype=torch.uint8, device="cuda")
        s = torch.empty(R, dtype=torch.float32, device="cuda")
        a = torch.empty(R, dtype=torch.bfloat16, device="cuda")
        col = torch.zeros(C, dtype=torch.float32, device="cuda")
        ws_bytes = lib.l8_cast_rowwise_workspace(R, C)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
        L.check(lib.l8_cast_rowwise(x.data_ptr(), R, C, ldx, q.data_ptr(), ldq, s.data_ptr(), a.data_ptr(),
                                    col.data_ptr(), ws.data_ptr(), ws_bytes, _stream()), "l8_cast_rowwise")
        xc = xb[:, :C].contiguous()
        wq, wsc, wa = oracle.cast_rowwise(xc)
        tag = (case, R, C, ldx, ldq)
        assert torch.equal(q.cpu()[:, :C], wq), tag
        assert (q.cpu()[:, C:] == FILL).all(), tag
        assert bits_equal(s.cpu(), wsc) and bits_equal(a.cpu(), wa), tag
        assert bits_equal(col.cpu(), oracle.col_amax(xc).float()), tag


def test_cast_transposed_sweep():
    lib, L = _lib()
    rng = random.Random(2)
    for case, (R, C, ldx) in enumerate(_shapes(rng, 50, 900, 3000, 8)):
        ldq = R + rng.choice([0, 0, 1, 7, 16, 33])          # any leading dimension: the kernel falls back to byte stores
        xb = _bf16_rows(rng, R, C, ldx, 1000 + case)
        x = xb.cuda()
        xc = xb[:, :C].contiguous()
        tag = (case, R, C, ldx, ldq)
        # column-wise scales
        col = torch.zeros(C, dtype=torch.float32, device="cuda")
        L.check(lib.l8_col_amax(x.data_ptr(), R, C, ldx, col.data_ptr(), _stream()), "l8_col_amax")
        q = torch.full((C, ldq), FILL, dtype=torch.uint8, device="cuda")
        s = torch.empty(C, dtype=torch.float32, device="cuda")
        L.check(lib.l8_cast_colwise_transposed(x.data_ptr(), R, C, ldx, col.data_ptr(), q.data_ptr(), ldq, s.data_ptr(),
                                               _stream()), "l8_cast_colwise_transposed")
        wq, wsc = oracle.cast_colwise_transposed(xc)
        assert torch.equal(q.cpu()[:, :R], wq), tag
        assert (q.cpu()[:, R:] == FILL).all(), tag
        assert bits_equal(s.cpu(), wsc), tag
        # one scale, both layouts
        amax = oracle.amax_of_amaxes(oracle.row_amax(xc))
        for transpose in (0, 1):
            rows, cols = (C, R) if transpose else (R, C)
            ld = cols + (ldq - R)
            if not transpose:
                ld = (ld + 7) // 8 * 8
            q = torch.full((rows, ld), FILL, dtype=torch.uint8, device="cuda")
            s1 = torch.empty(1, dtype=torch.float32, device="cuda")
            L.check(lib.l8_cast_tensorwise(x.data_ptr(), R, C, ldx, amax.cuda().data_ptr(), 0, transpose, q.data_ptr(), ld,
                                           s1.data_ptr(), _stream()), "l8_cast_tensorwise")
            wq, wsc = oracle.cast_tensorwise(xc, amax, transpose=bool(transpose))
            assert torch.equal(q.cpu()[:, :cols], wq), tag + (transpose,)
            assert (q.cpu()[:, cols:] == FILL).all(), tag + (transpose,)
            assert bits_equal(s1.cpu(), wsc.reshape(-1)), tag


def test_gemm_sweep_exact():
    """Integer-valued operands in [-2, 2] and power-of-two scales: every partial sum is exact, so the result is
    the integer product whatever the accumulation order; random M, N, K (multiples of 16), padded leading
    dimensions on all three matrices, every scale-mode combination, optional bias, every tile configuration."""
    lib, L = _lib()
    rng = random.Random(3)
    n_algo = lib.l8_gemm_algo_count()
    for case in range(60):
        M = rng.choice([1, 5, 31, 33, 255, 257, rng.randrange(1, 700)])
        N = rng.choice([1, 8, 24, 129, 256, 300, rng.randrange(1, 700)])
        K = 16 * rng.randrange(1, 40)
        lda, ldb, ldc = K + 16 * rng.choice([0, 1, 4]), K + 16 * rng.choice([0, 2]), N + rng.choice([0, 1, 2, 8, 9])
        algo = rng.randrange(0, n_algo + 1)
        g = torch.Generator().manual_seed(2000 + case)
        A = torch.randint(-2, 3, (M, lda), generator=g).float()
        B = torch.randint(-2, 3, (N, ldb), generator=g).float()
        sa_row, sb_row, with_bias = rng.random() < 0.6, rng.random() < 0.6, rng.random() < 0.4
        sa = torch.tensor([2.0 ** rng.randrange(-3, 3) for _ in range(M if sa_row else 1)])
        sb = torch.tensor([2.0 ** rng.randrange(-2, 2) for _ in range(N if sb_row else 1)])
        bias = torch.randint(-4, 5, (N,), generator=g).to(torch.bfloat16) if with_bias else None
        qa, qb = A.to(torch.float8_e4m3fn).cuda(), B.to(torch.float8_e4m3fn).cuda()
        sad, sbd = sa.cuda(), sb.cuda()
        biasd = bias.cuda() if with_bias else None
        out = torch.full((M, ldc), 7.0, dtype=torch.bfloat16, device="cuda")
        L.check(lib.l8_gemm_nt(qa.data_ptr(), qb.data_ptr(), M, N, K, lda, ldb, sad.data_ptr(), int(sa_row),
                               sbd.data_ptr(), int(sb_row), biasd.data_ptr() if with_bias else None,
                               out.data_ptr(), ldc, algo, _stream()), "l8_gemm_nt")
        want = (A[:, :K].double() @ B[:, :K].double().t()) * sa.double().reshape(-1, 1) * sb.double().reshape(1, -1)
        if with_bias:
            want = want + bias.double()
        tag = (case, M, N, K, lda, ldb, ldc, algo, sa_row, sb_row, with_bias)
        # the fp32 result is exact; the only rounding is the final one to bf16 (round-to-nearest-even, as torch's)
        got = out.cpu()
        assert torch.equal(got[:, :N].double(), want.float().to(torch.bfloat16).double()), tag
        assert (got[:, N:].float() == 7.0).all(), tag


def _padded(t, ld, fill=0.0):
    """[R, ld] device buffer holding t in its first columns; returns (buffer, view of the operand)."""
    buf = torch.full((t.shape[0], ld), fill, dtype=t.dtype, device="cuda")
    buf[:, : t.shape[1]] = t
    return buf


def test_fused_gate_kernels_with_padded_rows_equal_the_dense_call():
    """l8_swiglu_cast_rowwise / l8_swiglu_bwd_cast_rowwise with every operand in a buffer of its own leading
    dimension: identical bits to the call on dense operands (whose parity is covered elsewhere), and nothing
    written past column C.  Row lengths cover the register, LDS-column-maxima and 1024-thread variants."""
    from lingua_amd import ops
    lib, L = _lib()
    rng = random.Random(4)
    for case in range(24):
        R = rng.choice([1, 3, 40, rng.randrange(1, 300)])
        C = 8 * rng.choice([1, 33, 500, 1376, 2048, 2750, 3600, rng.randrange(1, 4100)])
        g = torch.Generator().manual_seed(3000 + case)
        h1 = (torch.randn(R, C, generator=g) * 2).to(torch.bfloat16).cuda()
        h3 = torch.randn(R, C, generator=g).to(torch.bfloat16).cuda()
        dh = (torch.randn(R, C, generator=g) * 0.05).to(torch.bfloat16).cuda()
        ld1, ld3, ldd, ldh, ldq = (C + 8 * rng.choice([0, 1, 4, 16]) for _ in range(5))
        b1, b3, bd = _padded(h1, ld1), _padded(h3, ld3), _padded(dh, ldd)
        tag = (case, R, C, ld1, ld3, ldd, ldh, ldq)
        # forward
        col_ref = torch.zeros(C, dtype=torch.float32, device="cuda")
        h_ref, q_ref, s_ref, a_ref = ops.swiglu_cast_rowwise(h1, h3, col_amax=col_ref)
        hb = torch.full((R, ldh), 7.0, dtype=torch.bfloat16, device="cuda")
        qb = torch.full((R, ldq), FILL, dtype=torch.uint8, device="cuda")
        s = torch.empty(R, dtype=torch.float32, device="cuda")
        a = torch.empty(R, dtype=torch.bfloat16, device="cuda")
        col = torch.zeros(C, dtype=torch.float32, device="cuda")
        ws_bytes = lib.l8_swiglu_workspace(R, C)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
        L.check(lib.l8_swiglu_cast_rowwise(b1.data_ptr(), b3.data_ptr(), R, C, ld1, ld3, hb.data_ptr(), ldh, qb.data_ptr(), ldq,
                                           s.data_ptr(), a.data_ptr(), col.data_ptr(), ws.data_ptr(), ws_bytes // 2, _stream()),
                "l8_swiglu_cast_rowwise")
        assert torch.equal(hb[:, :C].view(torch.int16), h_ref.view(torch.int16)) and (hb[:, C:].float() == 7.0).all(), tag
        assert torch.equal(qb[:, :C], q_ref.view(torch.uint8)) and (qb[:, C:] == FILL).all(), tag
        assert torch.equal(s, s_ref.reshape(-1)) and torch.equal(a.view(torch.int16), a_ref.reshape(-1).view(torch.int16)), tag
        assert torch.equal(col, col_ref), tag
        # backward
        if C > 32768:
            continue
        c1_ref, c3_ref = (torch.zeros(C, dtype=torch.float32, device="cuda") for _ in range(2))
        g1_ref, g3_ref, q1_ref, q3_ref, s1_ref, s3_ref = ops.swiglu_bwd_cast_rowwise(dh, h1, h3, c1_ref, c3_ref)
        g1b, g3b = (torch.full((R, ldh), 7.0, dtype=torch.bfloat16, device="cuda") for _ in range(2))
        q1b, q3b = (torch.full((R, ldq), FILL, dtype=torch.uint8, device="cuda") for _ in range(2))
        s1, s3 = (torch.empty(R, dtype=torch.float32, device="cuda") for _ in range(2))
        c1, c3 = (torch.zeros(C, dtype=torch.float32, device="cuda") for _ in range(2))
        L.check(lib.l8_swiglu_bwd_cast_rowwise(bd.data_ptr(), b1.data_ptr(), b3.data_ptr(), R, C, ldd, ld1, ld3,
                                               g1b.data_ptr(), g3b.data_ptr(), ldh, q1b.data_ptr(), q3b.data_ptr(), ldq,
                                               s1.data_ptr(), s3.data_ptr(), c1.data_ptr(), c3.data_ptr(),
                                               ws.data_ptr(), ws_bytes, _stream()), "l8_swiglu_bwd_cast_rowwise")
        for got, ref in ((g1b, g1_ref), (g3b, g3_ref)):
            assert torch.equal(got[:, :C].view(torch.int16), ref.view(torch.int16)) and (got[:, C:].float() == 7.0).all(), tag
        for got, ref in ((q1b, q1_ref), (q3b, q3_ref)):
            assert torch.equal(got[:, :C], ref.view(torch.uint8)) and (got[:, C:] == FILL).all(), tag
        assert torch.equal(s1, s1_ref.reshape(-1)) and torch.equal(s3, s3_ref.reshape(-1)), tag
        assert torch.equal(c1, c1_ref) and torch.equal(c3, c3_ref), tag


def test_fused_norm_kernels_with_padded_rows_equal_the_dense_call():
    from lingua_amd import ops
    lib, L = _lib()
    rng = random.Random(5)
    for case in range(24):
        R = rng.choice([1, 2, 70, rng.randrange(1, 1500)])
        C = 8 * rng.choice([1, 64, 256, 512, 1024, rng.randrange(1, 1025)])
        w_f32 = rng.random() < 0.5
        g = torch.Generator().manual_seed(4000 + case)
        x = (torch.randn(R, C, generator=g) * 3).to(torch.bfloat16).cuda()
        gy = (torch.randn(R, C, generator=g) * 0.05).to(torch.bfloat16).cuda()
        w = (1 + 0.1 * torch.randn(C, generator=g)).to(torch.float32 if w_f32 else torch.bfloat16).cuda()
        ldx, ldy, ldq, ldg, ldgx = (C + 8 * rng.choice([0, 1, 4, 16]) for _ in range(5))
        xb, gb = _padded(x, ldx), _padded(gy, ldg)
        tag = (case, R, C, w_f32, ldx, ldy, ldq, ldg, ldgx)
        col_ref = torch.zeros(C, dtype=torch.float32, device="cuda")
        y_ref, q_ref, s_ref, r_ref = ops.rmsnorm_cast_rowwise(x, w, 1e-5, col_amax=col_ref)
        yb = torch.full((R, ldy), 7.0, dtype=torch.bfloat16, device="cuda")
        qb = torch.full((R, ldq), FILL, dtype=torch.uint8, device="cuda")
        s, rstd = (torch.empty(R, dtype=torch.float32, device="cuda") for _ in range(2))
        col = torch.zeros(C, dtype=torch.float32, device="cuda")
        ws_bytes = lib.l8_rmsnorm_workspace(R, C)
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
        L.check(lib.l8_rmsnorm_cast_rowwise(xb.data_ptr(), w.data_ptr(), int(w_f32), R, C, ldx, 1e-5, yb.data_ptr(), ldy,
                                            qb.data_ptr(), ldq, s.data_ptr(), rstd.data_ptr(), col.data_ptr(),
                                            ws.data_ptr(), ws_bytes, _stream()), "l8_rmsnorm_cast_rowwise")
        assert torch.equal(yb[:, :C].view(torch.int16), y_ref.view(torch.int16)) and (yb[:, C:].float() == 7.0).all(), tag
        assert torch.equal(qb[:, :C], q_ref.view(torch.uint8)) and (qb[:, C:] == FILL).all(), tag
        assert torch.equal(s, s_ref.reshape(-1)) and torch.equal(rstd, r_ref.reshape(-1)) and torch.equal(col, col_ref), tag
        gx_ref, gw_ref = ops.rmsnorm_bwd(gy, x, w, r_ref)
        gxb = torch.full((R, ldgx), 7.0, dtype=torch.bfloat16, device="cuda")
        gw = torch.empty(C, dtype=torch.float32, device="cuda")
        wsb = lib.l8_rmsnorm_bwd_workspace(R, C)
        ws2 = torch.empty(max(wsb, 16), dtype=torch.uint8, device="cuda")
        L.check(lib.l8_rmsnorm_bwd(gb.data_ptr(), xb.data_ptr(), w.data_ptr(), int(w_f32), rstd.data_ptr(), R, C, ldg, ldx,
                                   gxb.data_ptr(), ldgx, gw.data_ptr(), ws2.data_ptr(), wsb, _stream()), "l8_rmsnorm_bwd")
        assert torch.equal(gxb[:, :C].view(torch.int16), gx_ref.view(torch.int16)) and (gxb[:, C:].float() == 7.0).all(), tag
        assert torch.equal(gw, gw_ref.reshape(-1)), tag
