"""CPU-only checks of the host side: the C ABI exports what the header
declares, argument validation happens before any launch, and the converter /
module mirror the reference interface (lingua/float8.py:134-191)."""
import ctypes
import os
import re

import pytest
import torch
from torch import nn

import lingua_amd
from lingua_amd import _lib, ops
from lingua_amd.float8 import Fp8Linear, convert_linears_to_fp8, named_replace

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "lingua_fp8.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(l8_\w+)\s*\(", header))
    assert {"l8_cast_rowwise", "l8_cast_tensorwise", "l8_cast_colwise_transposed", "l8_gemm_nt", "l8_col_amax",
            "l8_amax_reduce", "l8_version", "l8_last_error", "l8_device_check", "l8_cast_rowwise_workspace"} <= declared
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert declared == set(_lib.SIGNATURES)
    assert _lib.load().l8_version() >= 1


def test_argument_validation_happens_before_launch():
    lib = _lib.load()
    fake = 1 << 20  # never dereferenced: every call below must be rejected on the host
    assert lib.l8_gemm_nt(fake, fake, 4, 4, 8, 16, 16, fake, 1, fake, 1, None, fake, 4, 0, None) == -1
    assert "multiple of 16" in _lib.last_error()
    assert lib.l8_gemm_nt(fake, fake, 4, 4, 16, 16, 16, fake, 7, fake, 1, None, fake, 4, 0, None) == -1
    assert lib.l8_gemm_nt(fake, fake, 4, 4, 16, 16, 16, fake, 1, fake, 1, None, fake, 4, 99, None) == -1
    assert lib.l8_gemm_nt(None, fake, 4, 4, 16, 16, 16, fake, 1, fake, 1, None, fake, 4, 0, None) == -1
    assert lib.l8_gemm_nt(fake + 1, fake, 4, 4, 16, 16, 16, fake, 1, fake, 1, None, fake, 4, 0, None) == -1
    assert lib.l8_cast_rowwise(fake, 4, 12, 12, fake, 12, fake, None, None, None, 0, None) == -1
    assert lib.l8_cast_rowwise(fake, -1, 8, 8, fake, 8, fake, None, None, None, 0, None) == -1
    assert lib.l8_cast_tensorwise(fake, 4, 8, 8, None, 0, 0, fake, 8, fake, None) == -1
    assert lib.l8_cast_colwise_transposed(fake, 4, 8, 8, None, fake, 4, fake, None) == -1
    # a tile of the transposed casts (256 rows) must stay within 1 GiB
    assert lib.l8_cast_tensorwise(fake, 4, 8, 1 << 21, fake, 0, 1, fake, 16, fake, None) == -1
    assert "row stride too large" in _lib.last_error()
    assert lib.l8_cast_colwise_transposed(fake, 4, 8, 1 << 21, fake, fake, 16, fake, None) == -1
    assert "row stride too large" in _lib.last_error()
    # empty problems are accepted and do nothing
    assert lib.l8_cast_rowwise(None, 0, 8, 8, None, 8, None, None, None, None, 0, None) == 0
    # the column-amax by-product needs the workspace the library asks for
    assert lib.l8_cast_rowwise_workspace(64, 1024) > 0
    assert lib.l8_cast_rowwise(fake, 64, 1024, 1024, fake, 1024, fake, None, fake, None, 0, None) == -1
    assert "workspace" in _lib.last_error()
    assert lib.l8_gemm_nt(None, None, 0, 4, 16, 16, 16, None, 1, None, 1, None, None, 4, 0, None) == 0


def test_no_cpu_path():
    x = torch.zeros(4, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.cast_rowwise(x)
    lin = Fp8Linear(16, 8, bias=False, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError):
        lin(x)


class Block(nn.Module):
    def __init__(self):
        super().__init__()
        self.w1 = nn.Linear(8, 16, bias=False)
        self.w2 = nn.Linear(16, 8, bias=True)
        self.norm = nn.LayerNorm(8)


class Model(nn.Module):
    def __init__(self):
        super().__init__()
        self.tok_embeddings = nn.Embedding(10, 8)
        self.layers = nn.ModuleList([Block(), Block()])
        self.output = nn.Linear(8, 10, bias=False)


def test_unknown_recipe_raises_runtime_error():
    with pytest.raises(RuntimeError, match="Unknown float8 recipe 'tensorwise'"):
        convert_linears_to_fp8(Model(), "tensorwise", r"layers\.[0-9]+\.")


def test_converter_filter_identity_and_state_dict():
    with torch.device("meta"):
        m = Model()
    params_before = dict(m.named_parameters())
    keys_before = list(m.state_dict().keys())
    out = convert_linears_to_fp8(m, "rowwise", r"layers\.[0-9]+\.")
    assert out is m
    for i in range(2):
        for name in ("w1", "w2"):
            lin = getattr(m.layers[i], name)
            assert type(lin) is Fp8Linear and isinstance(lin, nn.Linear)
            assert lin.weight is params_before[f"layers.{i}.{name}.weight"]
            assert lin.weight.device.type == "meta"
        assert m.layers[i].w2.bias is params_before[f"layers.{i}.w2.bias"]
        assert m.layers[i].w1.bias is None
        assert type(m.layers[i].norm) is nn.LayerNorm
    assert type(m.output) is nn.Linear                       # excluded by the default filter
    assert type(m.tok_embeddings) is nn.Embedding
    assert list(m.state_dict().keys()) == keys_before
    assert {id(p) for p in m.parameters()} == {id(p) for p in params_before.values()}


def test_converting_twice_or_a_subclass_asserts():
    m = convert_linears_to_fp8(Model(), "rowwise", r"layers\.")
    with pytest.raises(AssertionError):
        convert_linears_to_fp8(m, "rowwise", r"layers\.")

    class MyLinear(nn.Linear):
        pass

    m2 = nn.Sequential(MyLinear(4, 4))
    with pytest.raises(AssertionError, match="MyLinear"):
        convert_linears_to_fp8(m2, "rowwise", "")
    # a subclass that the filter does not match is left alone
    assert convert_linears_to_fp8(m2, "rowwise", "nomatch") is m2


def test_root_linear_is_replaced_and_returned():
    lin = nn.Linear(8, 4, bias=True, dtype=torch.bfloat16)
    out = convert_linears_to_fp8(lin, "rowwise", "")
    assert type(out) is Fp8Linear and out is not lin
    assert out.weight is lin.weight and out.bias is lin.bias
    assert out.weight.dtype == torch.bfloat16 and (out.in_features, out.out_features) == (8, 4)


def test_named_replace_is_post_order_with_dotted_names():
    seen = []

    def fn(mod, name):
        seen.append(name)
        return mod

    m = Model()
    assert named_replace(fn, m) is m
    assert seen[-1] == ""
    assert seen.index("layers.0.w1") < seen.index("layers.0") < seen.index("layers")
    assert "layers.1.norm" in seen and "output" in seen


def test_public_names_match_reference_module():
    for name in ("EPS", "scale", "matmul", "Fp8LinearFn", "Fp8Linear", "named_replace", "convert_linears_to_fp8"):
        assert hasattr(lingua_amd, name)
    assert lingua_amd.EPS == 1e-12


def test_custom_op_fake_kernels_on_meta_tensors():
    """lingua_amd.custom_ops: shape-only implementations (what torch.compile traces with) need no GPU."""
    import torch
    from lingua_amd import custom_ops  # noqa: F401  (registers the operators)
    a = torch.empty((32, 64), dtype=torch.bfloat16, device="meta")
    w = torch.empty((48, 64), dtype=torch.bfloat16, device="meta")
    bias = torch.empty((48,), dtype=torch.bfloat16, device="meta")
    out, amax_w, col = torch.ops.lingua_amd.fp8_linear_fwd(a, w, bias, True, 0)
    assert out.shape == (32, 48) and out.dtype == torch.bfloat16
    assert amax_w.shape == (48, 1) and amax_w.dtype == torch.bfloat16
    assert col.shape == (64,) and col.dtype == torch.float32
    assert torch.ops.lingua_amd.fp8_linear_fwd(a, w, None, False, 0)[2].numel() == 0
    ga, gb, gbias = torch.ops.lingua_amd.fp8_linear_bwd(out, a, w, amax_w, col, True, True, True, True, 0)
    assert ga.shape == a.shape and gb.shape == w.shape and gbias.shape == (48,)
    ga, gb, gbias = torch.ops.lingua_amd.fp8_linear_bwd(out, a, w, amax_w, col, False, True, False, True, 0)
    assert ga.numel() == 0 and gb.shape == w.shape and gbias.numel() == 0


def test_which_problems_share_the_k_range_of_their_last_round():
    """Host-side decision of tile configuration 15 (no GPU needed): the K range of the last round's tiles is shared
    out only where the exchange of partial sums pays, and the split the rule describes covers every (tile, K tile)
    of the tail exactly once with every owner waiting only for a workgroup with a lower number."""
    lib = _lib.load()
    cus = 256
    # the step's three products on 256 compute units: only the K = 16384 one (688 tiles, 2.69 rounds) splits
    assert lib.l8_gemm_shares_k(11008, 4096, 16384, cus) == 8
    assert lib.l8_gemm_shares_k(4096, 11008, 16384, cus) == 8
    assert lib.l8_gemm_shares_k(16384, 11008, 4096, cus) == 0      # K loop too short to pay for the exchange
    assert lib.l8_gemm_shares_k(16384, 4096, 11008, cus) == 0      # 1024 tiles: four full rounds
    assert lib.l8_gemm_shares_k(4096, 6656, 8192, cus) == 8
    assert lib.l8_gemm_shares_k(3300, 5096, 6128, cus) == 4        # four XCDs have a tail tile, four have none
    assert lib.l8_gemm_shares_k(1024, 1024, 16384, cus) == 0       # less than one round: nothing to share
    assert lib.l8_gemm_shares_k(16384, 4096, 11008, 4) < 0         # bad argument

    def split(cnt, W, KT, write=8, fix=4, least=16):
        rounds, r = divmod(cnt, W)
        if rounds == 0 or r == 0:
            return None
        helpers = W - r
        m = (r + helpers - 1) // helpers
        piece = (KT + fix - m * write) // (m + 1)
        return None if piece < least else (r, helpers, KT - piece)

    for W in (1, 2, 5, 16, 32, 38):
        for cnt in range(1, 3 * W + 1):
            for KT in (1, 20, 47, 48, 64, 100, 128, 500):
                s = split(cnt, W, KT)
                got = lib.l8_gemm_shares_k(256 * 8 * cnt, 256, 128 * KT, 8 * W)
                assert got == (8 if s else 0), (cnt, W, KT)
                if not s:
                    continue
                r, helpers, cut = s
                assert 0 < cut < KT
                cover = {}
                for loc in range(W):
                    if loc < helpers:                      # helper: K tiles cut.. of tiles loc, loc + helpers, ...
                        for tt in range(loc, r, helpers):
                            for k in range(cut, KT):
                                assert (tt, k) not in cover
                                cover[(tt, k)] = loc
                    else:                                  # owner of tile loc - helpers: K tiles 0..cut-1
                        for k in range(cut):
                            assert (loc - helpers, k) not in cover
                            cover[(loc - helpers, k)] = loc
                assert len(cover) == r * KT
                assert all(cover[(tt, KT - 1)] < cover[(tt, 0)] for tt in range(r))


def test_build_refuses_a_persistent_gemm_kernel_that_uses_scratch():
    from lingua_amd import build
    ok = {"_ZN2l821gemm_nt_stream_kernelILi4ELb0ELb0EEEvNS_8GemmArgsE": {"VGPRs": 158, "AGPRs": 256, "ScratchSize": 0, "VGPRs Spill": 0},
          "_ZN2l814gemm_nt_kernelILi2ELi2ELi4ELi4ELi5ELi8ELi0EEEvNS_8GemmArgsE": {"ScratchSize": 36, "VGPRs Spill": 8}}
    build._check_usage(ok)   # the one-workgroup-per-tile kernels may spill outside their K loop
    for field in ("ScratchSize", "VGPRs Spill"):
        bad = {k: dict(v) for k, v in ok.items()}
        bad["_ZN2l821gemm_nt_stream_kernelILi4ELb0ELb0EEEvNS_8GemmArgsE"][field] = 12
        with pytest.raises(RuntimeError):
            build._check_usage(bad)
    # the memory-streaming kernels (casts, gate, norm) must not use scratch memory either
    spilled = {k: dict(v) for k, v in ok.items()}
    spilled["_ZN2l822cast_rowwise_wg_kernelILi6ELb1EEEvPKtlilPhlPfPtS5_i"] = {"VGPRs": 128, "ScratchSize": 8, "VGPRs Spill": 1}
    with pytest.raises(RuntimeError, match="streaming"):
        build._check_usage(spilled)
    # a check that finds nothing to check must fail too: no remark parsed at all, or one without the figures
    with pytest.raises(RuntimeError):
        build._check_usage({})
    with pytest.raises(RuntimeError):
        build._check_usage({"_ZN2l821gemm_nt_stream_kernelILi4ELb0ELb0EEEvNS_8GemmArgsE": {"VGPRs": 158, "AGPRs": 256}})
    # and the shipped build's record lists every instantiation of the persistent kernel
    usage_file = os.path.join(os.path.dirname(build.LIB_PATH), "build", "resource_usage.txt")
    if os.path.exists(usage_file):
        text = open(usage_file).read()
        for inst in ("ILi4ELb0ELb0E", "ILi4ELb1ELb0E", "ILi4ELb0ELb1E", "ILi8ELb0ELb0E", "ILi2ELb0ELb0E", "ILi16ELb0ELb0E"):
            assert "gemm_nt_stream_kernel" + inst in text, inst


def test_converter_drops_compiled_code_like_the_reference():
    """lingua/float8.py:187 resets the dynamo code caches after the swap ("force re-compile everything"): a
    module compiled before the conversion is traced again by its next call.  Runs on the CPU with a filter that
    matches nothing, so no Fp8Linear (GPU only) is executed."""
    import torch
    from lingua_amd import convert_linears_to_fp8
    traces = []

    def backend(gm, example_inputs):
        traces.append(len(traces))
        return gm.forward

    torch._dynamo.reset()
    model = torch.nn.Sequential(torch.nn.Linear(8, 8), torch.nn.ReLU())
    compiled = torch.compile(model, backend=backend)
    x = torch.randn(2, 8)
    compiled(x)
    compiled(x)
    assert len(traces) == 1                    # second call served from the code cache
    assert convert_linears_to_fp8(model, "rowwise", r"layers\.[0-9]+\.") is model
    compiled(x)
    assert len(traces) == 2                    # traced afresh after the conversion
    torch._dynamo.reset()


def test_scale_rule_switch_is_host_state_with_a_checked_argument():
    """l8_set_scale_rule / l8_get_scale_rule: host-only state, default = the correctly rounded quotient, unknown rules
    rejected with a message; the Python switch drops the quantised copies it holds."""
    import lingua_amd
    from lingua_amd import _lib, ops
    lib = _lib.load()
    assert lib.l8_get_scale_rule() == 0 and ops.get_scale_rule() == "divide"
    assert lib.l8_set_scale_rule(7) != 0 and b"unknown rule" in lib.l8_last_error()
    assert lib.l8_get_scale_rule() == 0
    try:
        lingua_amd.set_scale_rule("times_inverse")
        assert lib.l8_get_scale_rule() == 1 and lingua_amd.get_scale_rule() == "times_inverse"
        with pytest.raises(RuntimeError, match="unknown scale rule"):
            lingua_amd.set_scale_rule("fast")
        assert lingua_amd.get_scale_rule() == "times_inverse"
    finally:
        lingua_amd.set_scale_rule("divide")
    assert lib.l8_get_scale_rule() == 0


def test_linear_refuses_operands_it_cannot_serve_before_any_gpu_work():
    """No CPU path, bf16 only, feature counts in multiples of 16 (the reference gets the last one from
    torch._scaled_mm at lingua/float8.py:65): RuntimeError with the reason, raised before anything is launched."""
    from lingua_amd.float8 import Fp8LinearFn
    x = torch.zeros(8, 32, dtype=torch.bfloat16)
    w = torch.zeros(48, 32, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        Fp8LinearFn.apply(x, w, None)
    with pytest.raises(RuntimeError, match="bf16 input and weight required"):
        Fp8LinearFn.apply(x.float(), w, None)
    meta_x = torch.zeros(8, 40, dtype=torch.bfloat16, device="meta")
    with pytest.raises(RuntimeError):
        Fp8LinearFn.apply(meta_x, torch.zeros(48, 40, dtype=torch.bfloat16, device="meta"), None)


def test_a_named_library_that_is_not_there_fails_loudly():
    """LINGUA_FP8_LIB points lingua_amd at another build of the library (a tuning variant); a path that does not exist
    is an error that names the path, never a silent return to the shipped library."""
    import subprocess
    import sys
    code = ("import lingua_amd._lib as L\n"
            "try:\n    L.load()\nexcept RuntimeError as e:\n    print('RuntimeError', str(e))\n")
    env = dict(os.environ, LINGUA_FP8_LIB="/nonexistent/libl8_variant.so", PYTHONPATH=os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=120)
    assert "RuntimeError" in out.stdout and "/nonexistent/libl8_variant.so" in out.stdout, out.stdout + out.stderr
