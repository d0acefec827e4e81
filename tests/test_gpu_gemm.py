"""GPU parity of the fp8 NT GEMM: exact on integer-valued operands (pins the
matrix-core lane layout, tile edges and K tails), within rel-L2 <= 1e-3 of the
oracle's bf16(fp32-accumulated dequantised product) on random operands."""
import pytest
import torch

import oracle
from conftest import rel_l2, seeded_bf16

pytestmark = pytest.mark.gpu

TOL = 1e-3  # rel-L2 of bf16 outputs, from the benchmark specification


def n_algos():
    from lingua_amd import ops
    return len(ops.gemm_algos())


def fp8(t):
    return t.to(torch.float8_e4m3fn)


ALGOS = list(range(0, 17))
SHAPES_EXACT = [(1, 1, 16), (32, 32, 64), (256, 256, 128), (256, 256, 256), (300, 200, 144), (257, 513, 272),
                (64, 1000, 48), (1000, 24, 208), (512, 768, 240)]


@pytest.mark.parametrize("algo", ALGOS)
def test_exact_small_integer_operands(algo):
    from lingua_amd import ops
    if algo > n_algos():
        pytest.skip("no such tile configuration")
    g = torch.Generator().manual_seed(100 + algo)
    for (M, N, K) in SHAPES_EXACT:
        A = torch.randint(-1, 2, (M, K), generator=g).float()
        B = torch.randint(-1, 2, (N, K), generator=g).float()
        sa = torch.tensor([2.0 ** (i % 5 - 2) for i in range(M)]).reshape(M, 1)
        sb = torch.tensor([2.0 ** (i % 3) for i in range(N)]).reshape(N, 1)
        out = ops.gemm_nt(fp8(A).cuda(), fp8(B).cuda(), sa.cuda(), sb.cuda(), algo=algo)
        want = (A.double() @ B.double().t()) * sa.double() * sb.double().t()
        assert torch.equal(out.cpu().double(), want), (algo, M, N, K)


@pytest.mark.parametrize("algo", [0, 1, 2, 3, 11, 15])
def test_k_indexing_with_one_hot_operands(algo):
    # B[n] is one-hot at k = pi(n): C[m,n] = A[m, pi(n)] exactly, for any K (tails included)
    from lingua_amd import ops
    g = torch.Generator().manual_seed(5)
    for (M, N, K) in [(96, 400, 400), (130, 1040, 1040), (64, 2064, 2064), (300, 4096, 4096)]:
        A = torch.randint(-8, 9, (M, K), generator=g).float()
        pi = torch.randperm(K, generator=g)[:N]
        B = torch.zeros(N, K)
        B[torch.arange(N), pi] = 1.0
        one = torch.ones(1, 1)
        out = ops.gemm_nt(fp8(A).cuda(), fp8(B).cuda(), one.cuda(), one.cuda(), algo=algo)
        assert torch.equal(out.cpu().float(), A[:, pi]), (M, N, K)
        # and the mirrored case: one-hot A picks rows of B
        out2 = ops.gemm_nt(fp8(B).cuda(), fp8(A).cuda(), one.cuda(), one.cuda(), algo=algo)
        assert torch.equal(out2.cpu().float(), A[:, pi].t()), (M, N, K)


def random_fp8_bytes(shape, g):
    q = torch.randint(0, 256, shape, generator=g, dtype=torch.int32).to(torch.uint8)
    q[(q & 0x7F) == 0x7F] = 0x38
    return q


@pytest.mark.parametrize("algo", ALGOS)
def test_random_operands_vs_oracle(algo):
    from lingua_amd import ops
    if algo > n_algos():
        pytest.skip("no such tile configuration")
    g = torch.Generator().manual_seed(200 + algo)
    for (M, N, K) in [(384, 320, 512), (100, 72, 80), (513, 260, 1040)]:
        qa, qb = random_fp8_bytes((M, K), g), random_fp8_bytes((N, K), g)
        sa = torch.rand(M, 1, generator=g) + 0.5
        sb = torch.rand(N, 1, generator=g) + 0.5
        bias = (torch.randn(N, generator=g) * 50).to(torch.bfloat16)
        A, B = qa.cuda().view(torch.float8_e4m3fn), qb.cuda().view(torch.float8_e4m3fn)
        for sa_, sb_, b_ in ((sa, sb, None), (sa, sb, bias), (sa, sb[:1], None), (sa[:1], sb[:1], bias)):
            out = ops.gemm_nt(A, B, sa_.cuda(), sb_.cuda(), b_.cuda() if b_ is not None else None, algo=algo)
            want = oracle.gemm_nt(qa, qb, sa_, sb_, b_)
            assert rel_l2(out, want) <= TOL, (algo, M, N, K)


def test_output_leading_dimension_and_unaligned_n():
    from lingua_amd import ops
    g = torch.Generator().manual_seed(9)
    M, N, K = 70, 52, 96
    qa, qb = random_fp8_bytes((M, K), g), random_fp8_bytes((N, K), g)
    sa, sb = torch.ones(M, 1), torch.ones(N, 1)
    buf = torch.full((M, 64), 7.0, dtype=torch.bfloat16, device="cuda")
    out = buf[:, 4:4 + N]
    ops.gemm_nt(qa.cuda().view(torch.float8_e4m3fn), qb.cuda().view(torch.float8_e4m3fn), sa.cuda(), sb.cuda(), out=out)
    want = oracle.gemm_nt(qa, qb, sa, sb)
    assert rel_l2(out, want) <= TOL
    assert (buf[:, :4] == 7.0).all() and (buf[:, 4 + N:] == 7.0).all()  # nothing written outside the view


def test_config1_forward_product_full_vs_oracle():
    from lingua_amd import ops
    x = seeded_bf16((4096, 2048), 1.0, seed=0)
    w = seeded_bf16((2048, 2048), 0.02, seed=1)
    qx, sx, _ = ops.cast_rowwise(x.cuda())
    qw, sw, _ = ops.cast_rowwise(w.cuda())
    out = ops.gemm_nt(qx, qw, sx, sw)
    want = oracle.gemm_nt(qx.cpu().view(torch.uint8), qw.cpu().view(torch.uint8), sx.cpu(), sw.cpu())
    assert rel_l2(out, want) <= TOL


@pytest.mark.parametrize("mnk", [(16384, 11008, 4096), (16384, 4096, 11008), (11008, 4096, 16384)])
def test_7b_shapes_vs_library_matmul_and_oracle_rows(mnk):
    # full size: against torch's fp32 GPU matmul of the dequantised operands (an independent library routine),
    # and a sample of rows against the CPU oracle
    from lingua_amd import ops
    M, N, K = mnk
    g = torch.Generator(device="cuda").manual_seed(M + N)
    a = torch.randn(M, K, generator=g, device="cuda").to(torch.bfloat16)
    b = (torch.randn(N, K, generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    qa, sa, _ = ops.cast_rowwise(a)
    qb, sb, _ = ops.cast_rowwise(b)
    out = ops.gemm_nt(qa, qb, sa, sb)
    torch.backends.cuda.matmul.allow_tf32 = False
    ref = ((qa.float() * sa) @ (qb.float() * sb).t()).to(torch.bfloat16)
    assert rel_l2(out, ref) <= TOL
    rows = torch.arange(0, M, max(1, M // 48), device="cuda")[:48]
    want = oracle.gemm_nt(qa[rows].cpu().view(torch.uint8), qb.cpu().view(torch.uint8), sa[rows].cpu(), sb.cpu())
    assert rel_l2(out[rows], want) <= TOL


# Shapes for which tile configuration 15 shares the K range of the last round's tiles out between workgroups (long K, tile
# count a little above a multiple of the compute units; 256 compute units assumed, on other parts the same shapes
# may run unsplit and the assertions hold all the same): 16 x 26 tiles with 64 K tiles (every XCD splits: 20 tail
# tiles, 12 helpers with one or two pieces each), and 13 x 20 ragged tiles with 48 K tiles and a K tail (four XCDs
# have one tail tile and split it, four have none).
SHAPES_SHARED_K = [(4096, 6656, 8192), (3300, 5096, 6128)]
SHAPES_SHARED_K_RANDOM = SHAPES_SHARED_K + [(11008, 4096, 16384)]  # + a 7B wgrad shape: three pieces per helper


@pytest.mark.parametrize("mnk", SHAPES_SHARED_K)
def test_shared_k_range_exact_and_repeatable(mnk):
    # {-1, 0, 1} operands and power-of-two scales: every partial sum is exact in fp32, so the split product must
    # equal the unsplit one and the true one bit for bit; two calls must agree bit for bit as well
    from lingua_amd import _lib, ops
    M, N, K = mnk
    g = torch.Generator(device="cuda").manual_seed(K)
    A = torch.randint(-1, 2, (M, K), generator=g, device="cuda").float()
    B = torch.randint(-1, 2, (N, K), generator=g, device="cuda").float()
    sa = torch.tensor([2.0 ** (i % 5 - 2) for i in range(M)], device="cuda").reshape(M, 1)
    sb = torch.tensor([2.0 ** (i % 3) for i in range(N)], device="cuda").reshape(N, 1)
    qa, qb = fp8(A), fp8(B)
    out = ops.gemm_nt(qa, qb, sa, sb, algo=ops.GEMM_ALGO_SHARED_K)
    torch.backends.cuda.matmul.allow_tf32 = False
    want = ((A @ B.t()) * sa * sb.t()).to(torch.bfloat16)  # integer sums below 2^24: exact in fp32
    assert torch.equal(out, want)
    again = ops.gemm_nt(qa, qb, sa, sb, algo=ops.GEMM_ALGO_SHARED_K)
    assert torch.equal(out, again)
    # the entry point without a workspace never splits
    plain = torch.empty_like(out)
    code = _lib.load().l8_gemm_nt(qa.data_ptr(), qb.data_ptr(), M, N, K, K, K, sa.data_ptr(), ops.SCALE_ROW, sb.data_ptr(),
                                  ops.SCALE_ROW, None, plain.data_ptr(), N, 0, torch.cuda.current_stream().cuda_stream)
    _lib.check(code, "l8_gemm_nt")
    assert torch.equal(out, plain)


@pytest.mark.parametrize("mnk", SHAPES_SHARED_K_RANDOM)
def test_shared_k_range_random_operands(mnk):
    from lingua_amd import ops
    M, N, K = mnk
    g = torch.Generator().manual_seed(M)
    qa, qb = random_fp8_bytes((M, K), g).cuda(), random_fp8_bytes((N, K), g).cuda()
    sa = (torch.rand(M, 1, generator=g) + 0.5).cuda()
    sb = (torch.rand(1, 1, generator=g) + 0.5).cuda()   # scalar scale on the B side, as in dgrad
    A, B = qa.view(torch.float8_e4m3fn), qb.view(torch.float8_e4m3fn)
    out = ops.gemm_nt(A, B, sa, sb, algo=ops.GEMM_ALGO_SHARED_K)
    torch.backends.cuda.matmul.allow_tf32 = False
    ref = ((A.float() * sa) @ (B.float() * sb).t()).to(torch.bfloat16)
    assert rel_l2(out, ref) <= TOL
    rows = torch.arange(0, M, M // 24, device="cuda")[:24]
    want = oracle.gemm_nt(qa[rows].cpu(), qb.cpu(), sa[rows].cpu(), sb.cpu())
    assert rel_l2(out[rows], want) <= TOL
    assert torch.equal(out, ops.gemm_nt(A, B, sa, sb, algo=ops.GEMM_ALGO_SHARED_K))  # fixed order of the partial sums: repeatable bit for bit


def test_shared_k_range_gives_up_instead_of_hanging():
    # With a wait limit of zero polls an owner never sees its helper's partial sums: its tile must come out as
    # NaN (never as a wrong number), the kernel must still finish, and the next call with the normal limit is right.
    from lingua_amd import _lib, ops
    M, N, K = SHAPES_SHARED_K[0]
    g = torch.Generator(device="cuda").manual_seed(3)
    A = torch.randint(-1, 2, (M, K), generator=g, device="cuda").float()
    B = torch.randint(-1, 2, (N, K), generator=g, device="cuda").float()
    one = torch.ones(1, 1, device="cuda")
    qa, qb = fp8(A), fp8(B)
    want = (A @ B.t()).to(torch.bfloat16)
    lib = _lib.load()
    ops.gemm_nt(qa, qb, one, one, algo=ops.GEMM_ALGO_SHARED_K)   # makes the workspace if this is its first use
    before = ops.shared_k_tiles_given_up()
    _lib.check(lib.l8_gemm_set_wait_limit(0), "l8_gemm_set_wait_limit")
    try:
        out = ops.gemm_nt(qa, qb, one, one, algo=ops.GEMM_ALGO_SHARED_K)
        torch.cuda.synchronize()
    finally:
        _lib.check(lib.l8_gemm_set_wait_limit(1 << 18), "l8_gemm_set_wait_limit")
    bad = torch.isnan(out)
    gave_up = ops.shared_k_tiles_given_up() - before
    assert gave_up == int(bad.reshape(M // 256, 256, N // 256, 256).permute(0, 2, 1, 3).reshape(-1, 256 * 256).any(dim=1).sum())
    assert torch.equal(out[~bad], want[~bad])           # what is not poisoned is right
    if torch.cuda.get_device_properties(0).multi_processor_count == 256:
        tiles = bad.reshape(M // 256, 256, N // 256, 256).permute(0, 2, 1, 3).reshape(-1, 256 * 256)
        n_bad = int(tiles.all(dim=1).sum())
        assert n_bad == int(tiles.any(dim=1).sum())      # whole tiles, nothing partial
        assert n_bad == 8 * 20                           # the 20 tail tiles of each XCD
    assert torch.equal(ops.gemm_nt(qa, qb, one, one, algo=ops.GEMM_ALGO_SHARED_K), want)
    assert ops.shared_k_tiles_given_up() - before == gave_up      # the healthy call adds nothing


# The persistent kernel with a bias, on problems where a workgroup computes several tiles (scales and bias are
# requested afresh per tile while the stores of the tile before are still in flight): ragged edges in both
# directions, a K tail, 17 x 18 and 33 x 34 tiles.
SHAPES_BIAS_PERSISTENT = [(4100, 4360, 1040), (8200, 8456, 1040)]


@pytest.mark.parametrize("algo", [0, 12])
@pytest.mark.parametrize("mnk", SHAPES_BIAS_PERSISTENT)
def test_persistent_kernel_with_bias_exact_integer_operands(algo, mnk):
    from lingua_amd import ops
    M, N, K = mnk
    g = torch.Generator(device="cuda").manual_seed(M + algo)
    A = torch.randint(-1, 2, (M, K), generator=g, device="cuda").float()
    B = torch.randint(-1, 2, (N, K), generator=g, device="cuda").float()
    sa = torch.tensor([2.0 ** (i % 5 - 2) for i in range(M)], device="cuda").reshape(M, 1)
    sb = torch.tensor([2.0 ** (i % 3) for i in range(N)], device="cuda").reshape(N, 1)
    bias = torch.randint(-64, 65, (N,), generator=g, device="cuda").to(torch.bfloat16)  # integers: exact sums
    torch.backends.cuda.matmul.allow_tf32 = False
    prod = A @ B.t()  # integer sums below 2^24: exact in fp32
    for sa_, sb_ in ((sa, sb), (sa[:1], sb[:1]), (sa, sb[:1])):
        out = ops.gemm_nt(fp8(A), fp8(B), sa_, sb_, bias, algo=algo)
        want = (prod * sa_ * sb_.t() + bias.float()).to(torch.bfloat16)
        assert torch.equal(out, want), (algo, mnk, sa_.numel(), sb_.numel())
        # and the same bits as the plain one-workgroup-per-tile kernel
        assert torch.equal(out, ops.gemm_nt(fp8(A), fp8(B), sa_, sb_, bias, algo=5))


@pytest.mark.parametrize("algo", [0, 12])
def test_persistent_kernel_with_bias_random_operands_vs_oracle_rows(algo):
    from lingua_amd import ops
    for (M, N, K) in SHAPES_BIAS_PERSISTENT + [(16384, 4096, 4096)]:
        g = torch.Generator().manual_seed(M + N)
        qa, qb = random_fp8_bytes((M, K), g), random_fp8_bytes((N, K), g)
        sa = torch.rand(M, 1, generator=g) + 0.5
        sb = torch.rand(N, 1, generator=g) + 0.5
        bias = (torch.randn(N, generator=g) * 5e4).to(torch.bfloat16)   # the size of the products: it must show
        A, B = qa.cuda().view(torch.float8_e4m3fn), qb.cuda().view(torch.float8_e4m3fn)
        rows = torch.cat([torch.arange(0, M, max(1, M // 40))[:40], torch.arange(M - 6, M)])
        for sa_, sb_ in ((sa, sb), (sa[:1], sb[:1])):
            out = ops.gemm_nt(A, B, sa_.cuda(), sb_.cuda(), bias.cuda(), algo=algo)
            want = oracle.gemm_nt(qa[rows], qb, sa_[rows] if sa_.numel() == M else sa_, sb_, bias)
            assert rel_l2(out[rows.cuda()], want) <= TOL, (algo, M, N, K)
            plain = ops.gemm_nt(A, B, sa_.cuda(), sb_.cuda(), bias.cuda(), algo=5)
            assert rel_l2(out, plain) <= 1e-4, (algo, M, N, K)  # the whole matrix, against the plain kernel


def _scaled_mm_rowwise(qa, qb, sa, sb, bias=None):
    """The call of lingua/float8.py:65-73 (use_fast_accum=True branch): row-wise scales, bias, bf16 out."""
    return torch._scaled_mm(qa, qb.t(), scale_a=sa.reshape(-1, 1), scale_b=sb.reshape(1, -1), bias=bias,
                            out_dtype=torch.bfloat16, use_fast_accum=True)


@pytest.mark.parametrize("mnk", [(4096, 2048, 2048), (2048, 8192, 2048), (4100, 4368, 1040), (16384, 4096, 4096)])
def test_against_the_scaled_mm_call_the_reference_makes(mnk):
    """`torch._scaled_mm` with row-wise scales is what the reference's matmul() calls (lingua/float8.py:65-73); on this
    GPU it is the vendor library's kernel, an independent implementation on the same matrix instructions.  On the same
    quantised operands the two bf16 results must agree far inside the benchmark's tolerance.  Both deviate from the
    correctly rounded product in about 1 % of the elements, K = 128 or K = 16384 alike: the fp8 matrix instruction sums
    its 64 products with roughly 12 bits below the largest of them, which no kernel above it can change -- that, not
    the order of accumulation, is why rel-L2 against the fp32 oracle sits near 2e-4 on every shape."""
    from lingua_amd import ops
    M, N, K = mnk
    x = seeded_bf16((M, K), 1.0, seed=M)
    w = seeded_bf16((N, K), 0.02, seed=N + 1)
    bias = seeded_bf16((N,), 1.0, seed=3).cuda()
    qa, sa, _ = ops.cast_rowwise(x.cuda())
    qb, sb, _ = ops.cast_rowwise(w.cuda())
    try:
        ref = _scaled_mm_rowwise(qa, qb, sa, sb)
        ref_b = _scaled_mm_rowwise(qa, qb, sa, sb, bias)
    except (RuntimeError, NotImplementedError) as e:   # a PyTorch build without row-wise scaling on this GPU
        pytest.skip(f"torch._scaled_mm with row-wise scales is not available here: {e}")
    for algo in (0, 5):
        out = ops.gemm_nt(qa, qb, sa, sb, algo=algo)
        assert rel_l2(out, ref) <= 1e-4, (algo, mnk)
        assert (out != ref).float().mean().item() <= 5e-4, (algo, mnk)   # measured: 5e-6 of the elements
        out_b = ops.gemm_nt(qa, qb, sa, sb, bias, algo=algo)
        assert rel_l2(out_b, ref_b) <= 1e-4, (algo, mnk)
    # the deviation both share: against the fp32 oracle on a sample of rows
    rows = torch.arange(0, M, max(1, M // 32))[:32]
    want = oracle.gemm_nt(qa[rows.cuda()].cpu().view(torch.uint8), qb.cpu().view(torch.uint8), sa[rows.cuda()].cpu(), sb.cpu())
    assert rel_l2(ref[rows.cuda()], want) <= TOL and rel_l2(out[rows.cuda()], want) <= TOL
