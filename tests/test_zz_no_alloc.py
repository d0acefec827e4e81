"""l8_cast_rowwise_noalloc, the entry point for callers that cannot allocate device memory: through the C ABI
itself, against l8_cast_rowwise (caller-supplied workspace) on the same inputs -- e4m3 bytes, scales, row
amaxes and column amaxes bit for bit -- on two calls in a row, the second on a smaller input, so that whatever
the first call left in the static scratch array must not leak into the second."""
import pytest
import torch

import oracle
from conftest import seeded_bf16
from golden_util import bits_equal

pytestmark = pytest.mark.gpu


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _run(lib, check, x, noalloc, with_col=True):
    R, C = x.shape
    q = torch.zeros((R, C), dtype=torch.uint8, device="cuda")
    s = torch.zeros(R, dtype=torch.float32, device="cuda")
    a = torch.zeros(R, dtype=torch.bfloat16, device="cuda")
    col = torch.full((C,), 3e30, dtype=torch.float32, device="cuda") if with_col else None
    colp = col.data_ptr() if with_col else None
    if noalloc:
        check(lib.l8_cast_rowwise_noalloc(x.data_ptr(), R, C, x.stride(0), q.data_ptr(), C, s.data_ptr(), a.data_ptr(),
                                          colp, _stream()), "l8_cast_rowwise_noalloc")
    else:
        need = lib.l8_cast_rowwise_workspace(R, C) if with_col else 0
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device="cuda")
        check(lib.l8_cast_rowwise(x.data_ptr(), R, C, x.stride(0), q.data_ptr(), C, s.data_ptr(), a.data_ptr(),
                                  colp, ws.data_ptr() if need else None, need, _stream()), "l8_cast_rowwise")
    torch.cuda.synchronize()
    return q, s, a, col


def test_noalloc_equals_the_workspace_entry_point_on_two_calls_in_a_row():
    from lingua_amd import _lib
    lib = _lib.load()
    _lib.require_device(0)                                        # set-up: looks the scratch array's address up
    big = seeded_bf16((3000, 11008), std=1.0, seed=101)           # 512 workgroups: 11 MB of the 16 MiB array
    small = seeded_bf16((37, 1024), std=0.02, seed=102)           # 10 workgroups, different row length
    small[5] = 0.0
    for x in (big, small):                                        # the second call sees the first one's leftovers
        xd = x.cuda()
        got = _run(lib, _lib.check, xd, noalloc=True)
        want = _run(lib, _lib.check, xd, noalloc=False)
        for g, w, what in zip(got, want, ("bytes", "scales", "row amaxes", "column amaxes")):
            assert bits_equal(g, w), f"{tuple(x.shape)}: {what} differ between the two entry points"
        # and both are the oracle's
        qo, so, ao = oracle.cast_rowwise(x)
        assert torch.equal(got[0].cpu(), qo) and bits_equal(got[1].cpu(), so) and bits_equal(got[2].cpu(), ao)
        assert bits_equal(got[3].cpu(), oracle.col_amax(x).float())
    # without column amaxes no scratch is involved; a strided input goes through as well
    wide = seeded_bf16((64, 1536), seed=103).cuda()[:, 256:1280]
    got = _run(lib, _lib.check, wide, noalloc=True, with_col=False)
    want = _run(lib, _lib.check, wide, noalloc=False, with_col=False)
    assert bits_equal(got[0], want[0]) and bits_equal(got[1], want[1]) and bits_equal(got[2], want[2])


def test_noalloc_rejects_shapes_beyond_its_scratch_array():
    from lingua_amd import _lib
    lib = _lib.load()
    _lib.require_device(0)
    R, C = 600, 16896                                             # 512 workgroups x 16896 columns x 2 bytes > 16 MiB
    assert lib.l8_cast_rowwise_workspace(R, C) > 16 * 1024 * 1024
    x = torch.zeros((R, C), dtype=torch.bfloat16, device="cuda")
    q = torch.full((R, C), 0x55, dtype=torch.uint8, device="cuda")
    s = torch.zeros(R, dtype=torch.float32, device="cuda")
    col = torch.zeros(C, dtype=torch.float32, device="cuda")
    code = lib.l8_cast_rowwise_noalloc(x.data_ptr(), R, C, C, q.data_ptr(), C, s.data_ptr(), None, col.data_ptr(), _stream())
    assert code == -1 and "scratch" in _lib.last_error()
    torch.cuda.synchronize()
    assert (q == 0x55).all()                                      # nothing was launched
    # the same shape without column amaxes needs no scratch and is served
    code = lib.l8_cast_rowwise_noalloc(x.data_ptr(), R, C, C, q.data_ptr(), C, s.data_ptr(), None, None, _stream())
    assert code == 0
    torch.cuda.synchronize()
    assert (q == 0).all()
