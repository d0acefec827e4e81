"""Operands beyond 2^31 bytes / elements (64-bit addressing in every kernel) and replay of the
path from a captured HIP graph (the entry points allocate nothing and never synchronise)."""
import pytest
import torch

import oracle
from conftest import rel_l2
from golden_util import bits_equal

pytestmark = pytest.mark.gpu

R_BIG, C_BIG = 70000, 32768          # 2.29e9 elements: row 65536 starts at element 2^31


@pytest.fixture(scope="module")
def big_x():
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.empty((R_BIG, C_BIG), dtype=torch.bfloat16, device="cuda")
    for r0 in range(0, R_BIG, 10000):           # generated in slabs: the fp32 normal of the whole tensor would be 9 GB
        r1 = min(r0 + 10000, R_BIG)
        x[r0:r1] = torch.randn((r1 - r0, C_BIG), generator=g, device="cuda").to(torch.bfloat16)
    yield x
    del x
    torch.cuda.empty_cache()


ROWS = [0, 1, 65535, 65536, 65537, R_BIG - 1]


def test_rowwise_cast_beyond_2g_elements(big_x):
    from lingua_amd import ops
    col = torch.zeros(C_BIG, dtype=torch.float32, device="cuda")
    q, s, a = ops.cast_rowwise(big_x, col_amax=col)
    rows = torch.tensor(ROWS, device="cuda")
    qo, so, ao = oracle.cast_rowwise(big_x[rows].cpu())
    assert torch.equal(q[rows].cpu().view(torch.uint8), qo)
    assert bits_equal(s[rows].cpu().reshape(-1), so) and bits_equal(a[rows].cpu().reshape(-1), ao)
    assert torch.equal(col, big_x.abs().amax(dim=0).float())
    # every row: the largest magnitude code is 0x7E (448) for a non-zero finite row
    assert int((q.view(torch.uint8) & 0x7F).amax(dim=1).min()) == 0x7E


def test_transposed_cast_beyond_2g_elements(big_x):
    from lingua_amd import ops
    col = big_x.abs().amax(dim=0).float()
    qt, st = ops.cast_colwise_transposed(big_x, col)
    assert qt.shape == (C_BIG, R_BIG)
    cols = [0, 1, 777, C_BIG - 1]
    want_q, want_s, _ = oracle.cast_rowwise(big_x[:, cols].t().contiguous().cpu())
    assert torch.equal(qt[cols].cpu().view(torch.uint8), want_q)
    assert bits_equal(st[cols].cpu().reshape(-1), want_s)


def test_gemm_operand_beyond_2g_bytes(big_x):
    from lingua_amd import ops
    qa, sa, _ = ops.cast_rowwise(big_x)                        # A: 70000 x 32768 e4m3 = 2.29 GB
    g = torch.Generator(device="cuda").manual_seed(8)
    w = (torch.randn((520, C_BIG), generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    qb, sb, _ = ops.cast_rowwise(w)
    for algo in (0, 1, 3):
        out = ops.gemm_nt(qa, qb, sa, sb, algo=algo)
        rows = torch.tensor(ROWS + [40000], device="cuda")
        want = ((qa[rows].float() * sa[rows]) @ (qb.float() * sb).t()).to(torch.bfloat16)
        assert rel_l2(out[rows], want) <= 1e-3, algo
    # the large operand on the B side (wgrad-like: few output rows, long rows of B)
    out_t = ops.gemm_nt(qb, qa, sb, sa)
    assert rel_l2(out_t[:, rows], want.t()) <= 1e-3


def test_linear_step_replayed_from_a_graph():
    """Forward + backward of an Fp8Linear captured once and replayed with new data: every replay must
    equal the eager result for that data."""
    from lingua_amd import Fp8Linear
    torch.manual_seed(3)
    lin = Fp8Linear(512, 768, bias=True, device="cuda", dtype=torch.bfloat16)
    x_static = torch.zeros((96, 512), dtype=torch.bfloat16, device="cuda", requires_grad=True)
    g_static = torch.zeros((96, 768), dtype=torch.bfloat16, device="cuda")

    def step():
        lin.weight.grad = lin.bias.grad = x_static.grad = None
        y = lin(x_static)
        y.backward(g_static)
        return y.detach(), x_static.grad, lin.weight.grad, lin.bias.grad

    def fill(seed):
        gen = torch.Generator(device="cuda").manual_seed(seed)
        with torch.no_grad():
            x_static.copy_(torch.randn(x_static.shape, generator=gen, device="cuda").to(torch.bfloat16))
            g_static.copy_((torch.randn(g_static.shape, generator=gen, device="cuda") * 0.02).to(torch.bfloat16))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):               # warm-up outside the capture: one-time attribute calls, allocator pools
        fill(0)
        for _ in range(3):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    lin.weight.grad = lin.bias.grad = x_static.grad = None
    with torch.cuda.graph(graph):
        outs = step()
    for seed in (11, 12, 13):
        fill(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [t.clone() for t in outs]
        want = [t.clone() for t in step()]      # eager work between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert torch.equal(a.view(torch.int16), b.view(torch.int16)), seed
