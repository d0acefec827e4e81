#!/usr/bin/env python3
"""Benchmark of the fp8 row-wise linear path on one MI355X.

Workload (the configuration the headline metric is quoted on): Llama-7B-shaped
SwiGLU MLP, dim 4096, ffn 11008, 16384 tokens, forward + backward with every
linear in row-wise fp8 (forward, dgrad and wgrad on the fp8 matrix cores),
through the drop-in module API.  One "step" is one forward + backward of the
MLP = 9 GEMMs of 2*16384*4096*11008 flop = 13 297 218 748 416 flop.

Prints ONE JSON line.  `value` is TFLOP/s over whole steps (casts, SiLU and
autograd bookkeeping included) with inputs resident in HBM.  `roofline` is the
GEMM kernel alone, timed with events on its stream inside the timed steps.
`cpu_baseline` is the same recipe as PyTorch CPU ops on a token sample.  `sustained` is the same step run for
two seconds; `extras` holds side measurements (never part of `value`): the fused-gate path, torch._scaled_mm on
the step's GEMM shapes, one Fp8Linear forward+backward, the config-4 figures and the Llama-1B-shaped step.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

DIM, FFN, TOKENS = 4096, 11008, 16384
STEP_FLOP = 18 * TOKENS * DIM * FFN          # 9 GEMMs x 2*M*N*K
PEAK_FP8_TFLOPS = 5000.0                     # MI355X dense fp8 MFMA, published
PEAK_HBM_GBPS = 8000.0                       # MI355X HBM3E, published
# HBM-side bytes per GEMM launch come from rocprofv3 FETCH_SIZE / WRITE_SIZE runs, each scaled by what the same
# counter reads for a 256 MiB copy, mean over the three products the step launches three times each.  A counter run
# cannot share a process with the timed steps (it slows the kernels by ~8 %), so the figure is read from the
# committed summary of those runs (one line "roofline.traffic bytes per launch: N") and named as such in the line.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_nt_7b_hbm_traffic.txt")


def gemm_traffic_bytes():
    """The `roofline.traffic` figure and the kernel it was measured on, from the committed counter summary; a
    missing or unreadable summary is an error, not a silent constant."""
    import re
    with open(TRAFFIC_PROFILE) as f:
        text = f.read()
    m = re.search(r"^roofline\.traffic bytes per launch: (\d+)\s*$", text, re.M)
    k = re.search(r"^kernel: (\S+)\s*$", text, re.M)
    if not m or not k:
        raise RuntimeError(f"{TRAFFIC_PROFILE} holds no 'roofline.traffic bytes per launch:' / 'kernel:' line")
    return int(m.group(1)), k.group(1)


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=30)
    ap.add_argument("--algo", type=int, default=0, help="GEMM tile configuration (0 = library default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-sample-tokens", type=int, default=16384)
    ap.add_argument("--no-kernel-timing", action="store_true", help="do not record per-kernel events in the timed steps")
    ap.add_argument("--workload", choices=["mlp7b", "linear7b", "llama1b"], default="mlp7b",
                    help="mlp7b = the headline workload; linear7b = one 4096->11008 Fp8Linear forward+backward on 16384 "
                         "tokens (casts included); llama1b = full Llama-1B-shaped forward+backward step "
                         "(25 layers, dim 2048, ffn 8192, vocab 128256, 4 x 4096 tokens), reported in tokens/s")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the side measurements: the sustained leg, the fused-SwiGLU variant of the same MLP, "
                         "torch._scaled_mm (what the reference calls) on the step's GEMM shapes, one Fp8Linear, the "
                         "config-4 figures and the Llama-1B step")
    ap.add_argument("--sustained-seconds", type=float, default=2.0,
                    help="length of the sustained leg (same step, run for at least this long)")
    ap.add_argument("--gemm-shape", choices=["fwd", "dgrad", "wgrad"], default="fwd",
                    help="with --kernel-only gemm: which product of the 4096 -> 11008 linear (reduction 4096, 11008, 16384)")
    ap.add_argument("--launches", type=int, default=3, help="with --kernel-only gemm: number of launches")
    ap.add_argument("--kernel-only", choices=["gemm", "copy", "casts"], default=None,
                    help="profiling aid: launch only the forward-shape GEMM, or a plain 256 MiB device copy "
                         "(the reference point the FETCH_SIZE / WRITE_SIZE counters are scaled by), or each cast "
                         "kernel on its 7B-MLP shape, a few times")
    return ap.parse_args()


def make_mlp(torch, nn, dim, ffn, device):
    class SwiGLU(nn.Module):
        # layer names of lingua/transformer.py:430-471
        def __init__(self):
            super().__init__()
            self.w1 = nn.Linear(dim, ffn, bias=False)
            self.w3 = nn.Linear(dim, ffn, bias=False)
            self.w2 = nn.Linear(ffn, dim, bias=False)

        def forward(self, x):
            return self.w2(torch.nn.functional.silu(self.w1(x)) * self.w3(x))

    g = torch.Generator().manual_seed(0)
    m = SwiGLU().to(torch.bfloat16)
    with torch.no_grad():
        for p in m.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).to(torch.bfloat16))
    return m.to(device)


def cpu_baseline(torch, sample_tokens):
    """The recipe as PyTorch CPU ops (oracle/recipe_torch.py), on `sample_tokens` tokens of the same workload."""
    from oracle import recipe_torch as rt
    cores = os.cpu_count() or 1
    try:
        cores = len(os.sched_getaffinity(0))
    except Exception:
        pass
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(sample_tokens, DIM, generator=g).to(torch.bfloat16)
    gy = (torch.randn(sample_tokens, DIM, generator=g) * 1e-2).to(torch.bfloat16)
    w1 = (torch.randn(FFN, DIM, generator=g) * 0.02).to(torch.bfloat16)
    w3 = (torch.randn(FFN, DIM, generator=g) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn(DIM, FFN, generator=g) * 0.02).to(torch.bfloat16)
    t0 = time.perf_counter()
    rt.swiglu_mlp_fwd_bwd(x, w1, w2, w3, gy)
    dt = time.perf_counter() - t0
    flop = 18 * sample_tokens * DIM * FFN
    # configs[0], the reference's own CPU-runnable case: one row-wise linear forward, x [4096,2048], W [2048,2048]
    x1 = torch.randn(4096, 2048, generator=g).to(torch.bfloat16)
    w1c = (torch.randn(2048, 2048, generator=g) * 0.02).to(torch.bfloat16)
    reps = []
    for _ in range(4):
        t0 = time.perf_counter()
        rt.linear_forward(x1, w1c)
        reps.append(time.perf_counter() - t0)
    c1 = sorted(reps[1:])[1]   # median of three after one warm-up
    # configs[1]: Llama-1B-shaped SwiGLU MLP forward, 32768 tokens, one repetition
    x2 = torch.randn(32768, 2048, generator=g).to(torch.bfloat16)
    v1 = (torch.randn(8192, 2048, generator=g) * 0.02).to(torch.bfloat16)
    v3 = (torch.randn(8192, 2048, generator=g) * 0.02).to(torch.bfloat16)
    v2 = (torch.randn(2048, 8192, generator=g) * 0.02).to(torch.bfloat16)
    t0 = time.perf_counter()
    rt.linear_forward(torch.nn.functional.silu(rt.linear_forward(x2, v1)) * rt.linear_forward(x2, v3), v2)
    c2 = time.perf_counter() - t0
    del x2, v1, v2, v3
    # configs[3]: the 4096 -> 11008 linear on the outlier-stress activations, row-wise and tensor-wise, one repetition
    from bench_workloads import outlier_stress_input, seeded_bf16
    x4, _, _ = outlier_stress_input(rows=TOKENS, cols=DIM, seed=0)
    w4 = seeded_bf16((FFN, DIM), 0.02, seed=1)
    t0 = time.perf_counter()
    rt.linear_forward(x4, w4)
    rt.matmul(x4, x4.abs().amax().reshape(1, 1), w4, w4.abs().amax().reshape(1, 1))
    c4 = time.perf_counter() - t0
    del x4, w4
    # configs[4]: the seven fp8 linears of one Llama-1B block, forward + backward on the step's 16384 tokens, one repetition
    # (the block's attention, norms and the head are not part of the path and are left out; a step has 25 such blocks)
    t5 = 0.0
    for n_out, n_in, count in ((2048, 2048, 4), (8192, 2048, 2), (2048, 8192, 1)):
        a5 = torch.randn(TOKENS, n_in, generator=g).to(torch.bfloat16)
        g5 = (torch.randn(TOKENS, n_out, generator=g) * 1e-2).to(torch.bfloat16)
        w5 = (torch.randn(n_out, n_in, generator=g) * 0.02).to(torch.bfloat16)
        t0 = time.perf_counter()
        for _ in range(count):
            rt.linear_fwd_bwd(a5, w5, g5)
        t5 += time.perf_counter() - t0
    del a5, g5, w5
    flop5 = 6 * TOKENS * (4 * 2048 * 2048 + 3 * 2048 * 8192)
    return {
        "value": round(flop / dt / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"same MLP fwd+bwd on {sample_tokens} of {TOKENS} tokens, one repetition, {dt:.2f} s "
                  f"(PyTorch CPU ops: amax/clamp/div/reciprocal/mul/to(float8_e4m3fn), dequantise, fp32 matmul, bf16)",
        "config1_linear_forward": {"value": round(2 * 4096 * 2048 * 2048 / c1 / 1e12, 4), "unit": "TFLOP/s",
                                   "ms": round(c1 * 1e3, 2), "sample": "x [4096,2048] @ W [2048,2048]^T, casts included, median of 3"},
        "config2_mlp1b_forward": {"value": round(3 * 2 * 32768 * 2048 * 8192 / c2 / 1e12, 4), "unit": "TFLOP/s", "s": round(c2, 2),
                                  "sample": "Llama-1B-shaped SwiGLU MLP forward, 32768 tokens, one repetition"},
        "config4_outlier_stress_linear": {"value": round(2 * 2 * TOKENS * DIM * FFN / c4 / 1e12, 4), "unit": "TFLOP/s", "s": round(c4, 2),
                                          "sample": "4096 -> 11008 linear forward on the outlier-stress activations, row-wise + "
                                                    "tensor-wise, 16384 tokens, one repetition"},
        "config5_llama1b_block_linears": {"value": round(flop5 / t5 / 1e12, 4), "unit": "TFLOP/s", "s": round(t5, 2),
                                          "extrapolated_s_per_step": round(25 * t5, 1),
                                          "sample": "the 7 fp8 linears of ONE Llama-1B block (wq, wk, wv, wo, w1, w3, w2), forward + "
                                                    "backward, 16384 tokens, one repetition; extrapolated_s_per_step = 25 blocks x "
                                                    "this time, an extrapolation (linears only: no attention, norms, head or loss)"},
    }


def kernel_table(records):
    """{kernel: launches, avg_ms, and TFLOP/s (GEMM) or GB/s + fraction of HBM peak (everything else)} from the
    (name, start event, end event, algorithmic work) records of lingua_amd.ops.kernel_timer."""
    agg = {}
    for name, e0, e1, work in records:
        a = agg.setdefault(name, [0, 0.0, 0])
        a[0] += 1
        a[1] += e0.elapsed_time(e1)
        a[2] += work
    table = {}
    for name, (n, ms, work) in agg.items():
        if name == "gemm_nt":
            table[name] = {"launches": n, "avg_ms": round(ms / n, 4), "TFLOP/s": round(work / (ms * 1e-3) / 1e12, 1)}
        else:
            gbps = work / (ms * 1e-3) / 1e9
            table[name] = {"launches": n, "avg_ms": round(ms / n, 4), "GB/s": round(gbps, 1),
                           "frac_hbm": round(gbps / PEAK_HBM_GBPS, 4)}
    return table


def gemm_shape_table(torch, dev, iters=20, warm=5):
    """The GEMM alone on the products of the Llama-1B-shaped linears (dim 2048, ffn 8192, 16384 tokens:
    lingua/transformer.py:357-359,406,469-471 at that size; wq/wk/wv also as one fused product), of configs[0]
    and configs[1], and on the three 7B products: ms, TFLOP/s, fraction of the fp8 peak and the tile
    configuration the library picks, operands quantised from seeded normal data."""
    from lingua_amd import ops
    shapes = [("1B wq/wk/wv/wo fwd and dgrad", 16384, 2048, 2048), ("1B wq+wk+wv as one product, fwd", 16384, 6144, 2048),
              ("1B w1/w3 fwd, w2 dgrad", 16384, 8192, 2048), ("1B w2 fwd, w1/w3 dgrad", 16384, 2048, 8192),
              ("1B wq/wk/wv/wo wgrad", 2048, 2048, 16384), ("1B w1/w3 wgrad", 8192, 2048, 16384),
              ("1B w2 wgrad", 2048, 8192, 16384), ("config 1 linear fwd", 4096, 2048, 2048),
              ("config 2 w1/w3 fwd", 32768, 8192, 2048), ("config 2 w2 fwd", 32768, 2048, 8192),
              ("7B fwd", TOKENS, FFN, DIM), ("7B dgrad", TOKENS, DIM, FFN), ("7B wgrad", FFN, DIM, TOKENS)]
    g = torch.Generator(device=dev).manual_seed(11)
    rows = []
    for what, M, N, K in shapes:
        a = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
        b = (torch.randn(N, K, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        qa, sa, _ = ops.cast_rowwise(a)
        qb, sb, _ = ops.cast_rowwise(b)
        out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        for _ in range(warm):
            ops.gemm_nt(qa, qb, sa, sb, out=out)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            ops.gemm_nt(qa, qb, sa, sb, out=out)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / iters
        tf = 2 * M * N * K / (ms * 1e-3) / 1e12
        rows.append({"what": what, "M": M, "N": N, "K": K, "ms": round(ms, 4), "TFLOP/s": round(tf, 1),
                     "frac_of_fp8_peak": round(tf / PEAK_FP8_TFLOPS, 4), "kernel": ops.gemm_pick(M, N, K)[1]})
        del a, b, qa, qb, out
    return rows


def config_figures(torch, dev, iters=20, warm=5):
    """GPU figures for the configurations the CPU baseline also times: configs[0] (one row-wise linear forward,
    x [4096,2048], W [2048,2048], casts included), configs[1] (Llama-1B-shaped SwiGLU MLP forward, 32768 tokens,
    through convert_linears_to_fp8) and the configs[3] linear (4096 -> 11008 forward on 16384 outlier-stress
    tokens, row-wise and tensor-wise: casts + GEMM each)."""
    from torch import nn
    from lingua_amd import Fp8Linear, convert_linears_to_fp8, ops
    from bench_workloads import outlier_stress_input, seeded_bf16

    def clock(fn):
        for _ in range(warm):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / iters

    res = {}
    with torch.no_grad():
        lin = Fp8Linear(2048, 2048, bias=False, device=dev, dtype=torch.bfloat16)
        lin.weight.copy_(seeded_bf16((2048, 2048), 0.02, seed=1).to(dev))
        x1 = seeded_bf16((4096, 2048), 1.0, seed=0).to(dev)
        ms = clock(lambda: lin(x1))
        flop1 = 2 * 4096 * 2048 * 2048
        res["config1_linear_forward"] = {"ms": round(ms, 4), "TFLOP/s": round(flop1 / (ms * 1e-3) / 1e12, 1),
                                         "what": "x [4096,2048] @ W [2048,2048]^T, both casts + GEMM per call, eager: three "
                                                 "launches of 5-20 us each, so the host's launch path is what is timed"}
        # the same call replayed from a captured HIP graph: what the GPU needs for it
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            lin(x1)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_graph = lin(x1)
        ms = clock(graph.replay)
        assert torch.equal(y_graph, lin(x1))
        res["config1_linear_forward"]["graph_replay_ms"] = round(ms, 4)
        res["config1_linear_forward"]["graph_replay_TFLOP/s"] = round(flop1 / (ms * 1e-3) / 1e12, 1)
        del graph, y_graph
        mlp = make_mlp(torch, nn, 2048, 8192, dev)
        mlp = convert_linears_to_fp8(nn.ModuleDict({"layers": nn.ModuleList([mlp])}), "rowwise", r"layers\.[0-9]+\.")["layers"][0]
        x2 = seeded_bf16((32768, 2048), 1.0, seed=2).to(dev)
        ms = clock(lambda: mlp(x2))
        flop2 = 3 * 2 * 32768 * 2048 * 8192
        res["config2_mlp1b_forward"] = {"ms": round(ms, 4), "TFLOP/s": round(flop2 / (ms * 1e-3) / 1e12, 1),
                                        "frac_of_fp8_peak": round(flop2 / (ms * 1e-3) / 1e12 / PEAK_FP8_TFLOPS, 4),
                                        "what": "Llama-1B-shaped SwiGLU MLP forward, 32768 tokens: 3 GEMMs, 5 casts, silu and mul in bf16"}
        del mlp, x2, lin, x1
        torch.cuda.empty_cache()
        x4, _, _ = outlier_stress_input(rows=TOKENS, cols=DIM, seed=0)
        x4 = x4.to(dev)
        w4 = seeded_bf16((FFN, DIM), 0.02, seed=1).to(dev)

        def rowwise():
            qx, sx, _ = ops.cast_rowwise(x4)
            qw, sw, _ = ops.cast_rowwise(w4)
            return ops.gemm_nt(qx, qw, sx, sw)

        def tensorwise():
            _, _, ax = ops.cast_rowwise(x4, want_q=False)
            _, _, aw = ops.cast_rowwise(w4, want_q=False)
            qx, sx = ops.cast_tensorwise(x4, ops.amax_reduce(ax))
            qw, sw = ops.cast_tensorwise(w4, ops.amax_reduce(aw))
            return ops.gemm_nt(qx, qw, sx, sw)

        flop4 = 2 * TOKENS * DIM * FFN
        for name, fn in (("rowwise", rowwise), ("tensorwise", tensorwise)):
            ms = clock(fn)
            res["config4_linear_forward_" + name] = {"ms": round(ms, 4), "TFLOP/s": round(flop4 / (ms * 1e-3) / 1e12, 1),
                                                     "what": "4096 -> 11008 linear forward on 16384 outlier-stress tokens, "
                                                             + name + " scaling of both operands, amax + casts + GEMM per call"}
    return res


def extras(torch, mlp, timed, args):
    """Side measurements, never part of `value`:
    fused_swiglu     the same MLP, same recipe, through lingua_amd.swiglu.Fp8FeedForward (gate fused into the casts,
                     x quantised once for w1 and w3);
    torch_scaled_mm  torch._scaled_mm with row-wise scales -- the call the reference makes (lingua/float8.py:65-72) --
                     on the nine GEMM shapes of one step, same GPU; None where this PyTorch build refuses it."""
    from lingua_amd.swiglu import Fp8FeedForward
    res = {}
    fused = Fp8FeedForward(mlp.w1, mlp.w3, mlp.w2)
    dt = timed(fused, None)
    res["fused_swiglu"] = {"value": round(STEP_FLOP / (dt / args.steps) / 1e12, 2), "unit": "TFLOP/s",
                           "ms_per_step": round(dt / args.steps * 1e3, 4)}
    if not args.no_kernel_timing:
        # the fused gate kernels' own rates: a second pass with every launch bracketed (not part of the figure above)
        rec = []
        timed(fused, rec, {"swiglu_cast_rowwise", "swiglu_bwd_cast_rowwise"})
        res["fused_swiglu"]["kernels"] = kernel_table(rec)
    try:
        dev = mlp.w1.weight.device
        total_ms = 0.0
        for (M, N, K), count in (((TOKENS, FFN, DIM), 3), ((TOKENS, DIM, FFN), 3), ((FFN, DIM, TOKENS), 3)):
            a = torch.randn(M, K, device=dev).to(torch.float8_e4m3fn)
            b = torch.randn(N, K, device=dev).to(torch.float8_e4m3fn)
            sa = torch.ones(M, 1, device=dev)
            sb = torch.ones(1, N, device=dev)
            for _ in range(5):
                torch._scaled_mm(a, b.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(10):
                torch._scaled_mm(a, b.t(), scale_a=sa, scale_b=sb, out_dtype=torch.bfloat16)
            e1.record()
            torch.cuda.synchronize()
            total_ms += count * e0.elapsed_time(e1) / 10
        res["torch_scaled_mm"] = {"avg_ms": round(total_ms / 9, 4), "TFLOP/s": round(STEP_FLOP / (total_ms * 1e-3) / 1e12, 1),
                                  "what": "hipBLASLt through torch._scaled_mm, row-wise scales, mean over the step's 9 GEMMs"}
    except Exception as exc:  # not every PyTorch build has the row-wise kernel
        res["torch_scaled_mm"] = None
        res["torch_scaled_mm_error"] = str(exc)[:200]
    return res


def more_extras(torch, dev, args):
    """The other measurements of the benchmark, each freed before the next: one Fp8Linear forward+backward, the
    config-4 outlier-stress figures (row-wise against tensor-wise scaling) and the Llama-1B-shaped step."""
    res = {}
    res["linear7b"] = measure_linear7b(args, torch, dev)
    torch.cuda.empty_cache()
    res["gemm_shapes"] = gemm_shape_table(torch, dev)
    torch.cuda.empty_cache()
    res.update(config_figures(torch, dev))
    torch.cuda.empty_cache()
    from bench_workloads import outlier_stress_figures
    fig, tensors = outlier_stress_figures(TOKENS)
    del tensors
    torch.cuda.empty_cache()
    res["config4_outlier_stress"] = dict(fig, what="4096->11008 linear on Student-t(3) activations, 0.1 % of channels x100, "
                                         "1 % zero rows: SNR of the quantised x and rel-L2 of y against the fp32 product")
    res["parity"] = parity_figures(torch, dev)
    torch.cuda.empty_cache()
    res["llama1b"] = measure_llama1b(torch, dev, steps=5, warmup=2, fused_too=True)
    return res


def parity_figures(torch, dev):
    """Not a timing: how this library's results sit beside what PyTorch itself computes on this GPU for configs[0]
    (x [4096,2048] ~ N(0,1), W [2048,2048] ~ N(0,0.02^2), seed 0).  (1) the product against torch._scaled_mm with
    row-wise scales -- the call the reference makes -- on the same quantised operands; (2) the two readings of
    `clamp(amax) / 448`: the correctly rounded quotient (ATen's CPU kernel, this library's default) against the product
    with fp32(1/448) (ATen's GPU kernel): scales and bytes that differ, and what that does to y."""
    import lingua_amd
    from lingua_amd import ops
    from bench_workloads import seeded_bf16, rel_l2
    x = seeded_bf16((4096, 2048), 1.0, seed=0).to(dev)
    w = seeded_bf16((2048, 2048), 0.02, seed=1).to(dev)
    out = {}
    qx, sx, _ = ops.cast_rowwise(x)
    qw, sw, _ = ops.cast_rowwise(w)
    y = ops.gemm_nt(qx, qw, sx, sw)
    try:
        ref = torch._scaled_mm(qx, qw.t(), scale_a=sx.reshape(-1, 1), scale_b=sw.reshape(1, -1), out_dtype=torch.bfloat16,
                               use_fast_accum=True)
        out["gemm_vs_torch_scaled_mm"] = {"rel_l2": float(f"{rel_l2(y, ref):.3e}"),
                                          "elements_differing": float(f"{(y != ref).float().mean().item():.3e}")}
    except (RuntimeError, NotImplementedError) as exc:
        out["gemm_vs_torch_scaled_mm"] = {"error": str(exc)[:200]}
    try:
        lingua_amd.set_scale_rule("times_inverse")
        qx2, sx2, _ = ops.cast_rowwise(x)
        qw2, sw2, _ = ops.cast_rowwise(w)
        y2 = ops.gemm_nt(qx2, qw2, sx2, sw2)
        # PyTorch's own kernels on this GPU, op for op as lingua/float8.py:43-47 issues them
        s_t = torch.clamp(x.abs().amax(dim=-1, keepdim=True).float(), min=1e-12) / 448.0
        q_t = (x * s_t.reciprocal()).to(torch.float8_e4m3fn)
    finally:
        lingua_amd.set_scale_rule("divide")
    out["division_rule"] = {
        "scales_differing": round((sx.view(torch.int32) != sx2.view(torch.int32)).float().mean().item(), 4),
        "bytes_differing": float(f"{(qx.view(torch.uint8) != qx2.view(torch.uint8)).float().mean().item():.3e}"),
        "rel_l2_of_y_between_rules": float(f"{rel_l2(y2, y):.3e}"),
        "times_inverse_equals_torch_gpu_ops": bool(torch.equal(q_t.view(torch.uint8), qx2.view(torch.uint8))
                                                   and torch.equal(s_t.view(torch.int32), sx2.view(torch.int32))),
        "divide_equals_torch_gpu_ops": bool(torch.equal(q_t.view(torch.uint8), qx.view(torch.uint8))
                                            and torch.equal(s_t.view(torch.int32), sx.view(torch.int32))),
    }
    return out


def bump_versions(torch, params):
    """What an optimizer step does to the parameters as far as this library can see: their version counters
    advance (no device work), so nothing keyed on a weight's version can be reused from the step before."""
    for p in params:
        torch.autograd.graph.increment_version(p)


def measure_linear7b(args, torch, dev):
    """One Fp8Linear 4096 -> 11008 on 16384 tokens, forward + backward (dgrad + fp8 wgrad), casts included."""
    from lingua_amd import Fp8Linear
    g = torch.Generator().manual_seed(0)
    lin = Fp8Linear(DIM, FFN, bias=False, device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_((torch.randn(FFN, DIM, generator=g) * 0.02).to(torch.bfloat16))
    x = torch.randn(TOKENS, DIM, generator=g).to(torch.bfloat16).to(dev).requires_grad_(True)
    gy = (torch.randn(TOKENS, FFN, generator=g) * 1e-2).to(torch.bfloat16).to(dev)

    def step():
        lin.weight.grad = x.grad = None
        bump_versions(torch, [lin.weight])
        lin(x).backward(gy)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    flop = 6 * TOKENS * DIM * FFN
    return {"value": round(flop / dt / 1e12, 2), "unit": "TFLOP/s", "ms_per_step": round(dt * 1e3, 4),
            "frac_of_fp8_peak": round(flop / dt / 1e12 / PEAK_FP8_TFLOPS, 4), "flop_per_step": flop,
            "what": "single Fp8Linear 4096->11008 fwd+bwd (dgrad + fp8 wgrad), 16384 tokens, casts included"}


def run_linear7b(args, torch, dev):
    r = measure_linear7b(args, torch, dev)
    print(json.dumps({
        "metric": "fp8 rowwise linear fwd+bwd TFLOP/s, one 4096->11008 linear", "value": r["value"],
        "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": r["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3fn", "data": "synthetic",
        "config": {"workload": r["what"], "flop_per_step": r["flop_per_step"]},
        "frac_of_fp8_peak": r["frac_of_fp8_peak"],
    }))


def measure_llama1b(torch, dev, steps, warmup, fused_too=True):
    """configs[4]: tokens/s of a Llama-1B-shaped forward+backward step, block linears in row-wise fp8."""
    from lingua_amd import convert_linears_to_fp8
    from bench_workloads import Llama, LLAMA_1B, llama_flops_per_token
    B, S = 4, 4096
    with torch.device(dev):
        model = Llama(**LLAMA_1B).to(torch.bfloat16)
    model.init_weights(0.02, seed=0)
    model = convert_linears_to_fp8(model, "rowwise", r"layers\.[0-9]+\.")
    g = torch.Generator().manual_seed(0)
    tokens = torch.randint(0, LLAMA_1B["vocab"], (B, S), generator=g).to(dev)
    labels = torch.randint(0, LLAMA_1B["vocab"], (B, S), generator=g).to(dev)

    def timed(m):
        params = list(m.parameters())

        def step():
            for p in params:
                p.grad = None
            bump_versions(torch, params)
            m(tokens, labels).backward()

        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / steps

    dt = timed(model)

    def kernel_share(m, step_dt):
        """Two more steps with every launch of this library bracketed by events: the share of the step's time that
        its kernels account for (the rest is the stand-in model's plain PyTorch: attention, rope, embeddings, loss,
        residual adds, and the bf16 output head), and the kernels' own table."""
        from lingua_amd import ops
        params = list(m.parameters())
        rec = []
        ops.kernel_timer, ops.kernel_timer_names = rec, None
        try:
            for _ in range(2):
                for p in params:
                    p.grad = None
                bump_versions(torch, params)
                m(tokens, labels).backward()
            torch.cuda.synchronize()
        finally:
            ops.kernel_timer, ops.kernel_timer_names = None, None
        table = kernel_table(rec)
        ms = sum(e0.elapsed_time(e1) for _, e0, e1, _ in rec) / 2
        gemm_ms = sum(e0.elapsed_time(e1) for name, e0, e1, _ in rec if name == "gemm_nt") / 2
        return {"fp8_kernels_ms_per_step": round(ms, 3), "fp8_gemm_ms_per_step": round(gemm_ms, 3),
                "share_of_step": round(ms / (step_dt * 1e3), 4), "kernels": table}

    share = kernel_share(model, dt)
    fused_dt = None
    if fused_too:
        # same weights, gate fused into the casts, norms that hand their output over quantised, one product for wq/wk/wv
        from lingua_amd.norm import fuse_rmsnorm
        from lingua_amd.qkv import fuse_qkv
        from lingua_amd.swiglu import fuse_feed_forward
        fused_dt = timed(fuse_qkv(fuse_rmsnorm(fuse_feed_forward(model))))
    fpt = llama_flops_per_token(LLAMA_1B["n_layers"], LLAMA_1B["dim"], LLAMA_1B["ffn_dim"], LLAMA_1B["vocab"], S)
    fp8_flop = 25 * 3 * (4 * 2 * B * S * 2048 * 2048 + 3 * 2 * B * S * 2048 * 8192)
    res = {"value": round(B * S / dt, 1), "unit": "tokens/s", "ms_per_step": round(dt * 1e3, 3), "steps": steps, "warmup": warmup,
           "model_TFLOP/s": round(fpt * B * S / dt / 1e12, 1), "fp8_linear_TFLOP/s_if_alone": round(fp8_flop / dt / 1e12, 1),
           "what": "Llama-1B-shaped step fwd+bwd (configs[4]): 25 layers, dim 2048, ffn 8192, vocab 128256, 4 x 4096 tokens; "
                   "block linears through convert_linears_to_fp8, the rest of the step is the stand-in model's plain PyTorch"}
    res["fp8_path"] = share
    if fused_dt is not None:
        res["fused_swiglu_and_rmsnorm"] = {"value": round(B * S / fused_dt, 1), "unit": "tokens/s",
                                           "ms_per_step": round(fused_dt * 1e3, 3)}
    del model
    torch.cuda.empty_cache()
    return res


def run_llama1b(args, torch, dev):
    from bench_workloads import LLAMA_1B
    r = measure_llama1b(torch, dev, args.steps, args.warmup, fused_too=not args.no_extras)
    print(json.dumps({
        "metric": "Llama-1B forward+backward tokens/s, block linears fp8 row-wise", "value": r["value"],
        "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": r["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "fp8_e4m3fn", "data": "synthetic",
        "config": {"workload": "llama-1B step fwd+bwd (configs[4])", "batch": 4, "seq_len": 4096, **LLAMA_1B},
        "model_TFLOP/s": r["model_TFLOP/s"],
        "fp8_linear_TFLOP/s_if_alone": r["fp8_linear_TFLOP/s_if_alone"],
        "fp8_path": r["fp8_path"],
        "extras": {"fused_swiglu_and_rmsnorm": r.get("fused_swiglu_and_rmsnorm")},
    }))


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build runs on exactly one GPU (no collectives are part of the fp8 linear path); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from torch import nn
    from lingua_amd import convert_linears_to_fp8, ops
    from lingua_amd import float8 as f8

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    f8.config.gemm_algo = args.algo

    if args.kernel_only == "copy":
        n = 256 << 20
        src = torch.ones(n, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"kernel_only": "copy", "bytes_read": n, "bytes_written": n, "launches": 3}))
        return
    if args.kernel_only == "gemm":
        M, N, K = {"fwd": (TOKENS, FFN, DIM), "dgrad": (TOKENS, DIM, FFN), "wgrad": (FFN, DIM, TOKENS)}[args.gemm_shape]
        g = torch.Generator().manual_seed(2)
        a = torch.randn(M, K, generator=g).to(torch.bfloat16).to(dev)
        b = (torch.randn(N, K, generator=g) * 0.02).to(torch.bfloat16).to(dev)
        qa, sa, _ = ops.cast_rowwise(a)
        qb, sb, _ = ops.cast_rowwise(b)
        out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        warm = min(10, args.launches // 2)   # launches before the timed ones (the clock settles under load)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for i in range(args.launches):
            if i == warm:
                e0.record()
            ops.gemm_nt(qa, qb, sa, sb, algo=args.algo, out=out)
        e1.record()
        torch.cuda.synchronize()
        avg_ms = e0.elapsed_time(e1) / (args.launches - warm)
        print(json.dumps({"kernel_only": "gemm", "M": M, "N": N, "K": K, "launches": args.launches,
                          "avg_ms": round(avg_ms, 4), "TFLOP/s": round(2 * M * N * K / avg_ms / 1e9, 1),
                          "flop_per_launch": 2 * M * N * K,
                          "algorithmic_bytes": M * K + N * K + 2 * M * N + 4 * (M + N)}))
        return

    if args.kernel_only == "casts":
        g = torch.Generator().manual_seed(3)
        x = torch.randn(TOKENS, DIM, generator=g).to(torch.bfloat16).to(dev)
        h1 = torch.randn(TOKENS, FFN, generator=g).to(torch.bfloat16).to(dev)
        h3 = torch.randn(TOKENS, FFN, generator=g).to(torch.bfloat16).to(dev)
        w = (torch.randn(FFN, DIM, generator=g) * 0.02).to(torch.bfloat16).to(dev)
        amax_w = ops.amax_reduce(ops.cast_rowwise(w, want_q=False)[2])
        col_x = ops.col_amax(x)
        col_h = ops.col_amax(h1)
        torch.cuda.synchronize()
        for _ in range(3):
            ops.cast_rowwise(x, col_amax=torch.zeros(DIM, dtype=torch.float32, device=dev))
            ops.cast_rowwise(h1, col_amax=torch.zeros(FFN, dtype=torch.float32, device=dev))
            ops.cast_rowwise(w)
            ops.cast_colwise_transposed(x, col_x)
            ops.cast_colwise_transposed(h1, col_h)
            ops.cast_tensorwise(w, amax_w, transpose=True)
            ops.swiglu_cast_rowwise(h1, h3, want_h=True, col_amax=torch.zeros(FFN, dtype=torch.float32, device=dev))
            ops.swiglu_bwd_cast_rowwise(h1, h3, h1, torch.zeros(FFN, dtype=torch.float32, device=dev),
                                        torch.zeros(FFN, dtype=torch.float32, device=dev))
        torch.cuda.synchronize()
        e = TOKENS * FFN
        print(json.dumps({"kernel_only": "casts", "launches_each": 3, "compulsory_bytes": {
            "cast_rowwise x[16384,4096] + col amax": TOKENS * DIM * 3 + 4 * TOKENS + 4 * DIM,
            "cast_rowwise h[16384,11008] + col amax": e * 3 + 4 * TOKENS + 4 * FFN,
            "cast_rowwise w[11008,4096]": FFN * DIM * 3 + 4 * FFN,
            "cast_colwise_transposed x": TOKENS * DIM * 3 + 4 * DIM,
            "cast_colwise_transposed h": e * 3 + 4 * FFN,
            "cast_tensorwise transposed w": FFN * DIM * 3 + 4,
            "swiglu_cast_rowwise (h written)": e * 7 + 4 * TOKENS + 4 * FFN,
            "swiglu_bwd_cast_rowwise": e * 12 + 8 * TOKENS + 8 * FFN}}))
        return

    if args.workload == "llama1b":
        run_llama1b(args, torch, dev)
        return
    if args.workload == "linear7b":
        run_linear7b(args, torch, dev)
        return

    mlp = make_mlp(torch, nn, DIM, FFN, dev)
    model = convert_linears_to_fp8(nn.ModuleDict({"layers": nn.ModuleList([mlp])}), "rowwise", r"layers\.[0-9]+\.")
    mlp = model["layers"][0]
    g = torch.Generator().manual_seed(1)
    x = torch.randn(TOKENS, DIM, generator=g).to(torch.bfloat16).to(dev).requires_grad_(True)
    gy = (torch.randn(TOKENS, DIM, generator=g) * 1e-2).to(torch.bfloat16).to(dev)

    def make_step(module):
        params = list(module.parameters())

        def step():
            for p in params:
                p.grad = None
            x.grad = None
            bump_versions(torch, params)   # as after an optimizer step: nothing may be reused from the step before
            y = module(x)
            y.backward(gy)
        return step

    def timed(module, records, names=None):
        step = make_step(module)
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        ops.kernel_timer, ops.kernel_timer_names = records, names
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
        ops.kernel_timer, ops.kernel_timer_names = None, None
        return elapsed

    def sustained(module, seconds):
        """The same step, repeated for at least `seconds` of wall clock: the clock the part settles at under load."""
        step = make_step(module)
        n, t0 = 0, time.perf_counter()
        while True:
            for _ in range(20):
                step()
            n += 20
            torch.cuda.synchronize()
            el = time.perf_counter() - t0
            if el >= seconds:
                return {"value": round(STEP_FLOP * n / el / 1e12, 2), "unit": "TFLOP/s", "steps": n, "seconds": round(el, 2),
                        "ms_per_step": round(el / n * 1e3, 4)}

    # Inside the timed steps only the GEMM launches (the roofline kernel) are bracketed by events: a pair of events
    # around every launch of the step costs 2.6 % of the step's time (measured), around the nine GEMMs 0.8 %.  The
    # cast kernels' table comes from a second, untimed-for-`value` pass with every launch bracketed.
    records = None if args.no_kernel_timing else []
    dt = timed(mlp, records, {"gemm_nt"})
    if records is not None:
        cast_records = []
        timed(mlp, cast_records)
        records += [r for r in cast_records if r[0] != "gemm_nt"]

    ms_per_step = dt / args.steps * 1e3
    tflops = STEP_FLOP / (dt / args.steps) / 1e12

    roofline = None
    kernels = {}
    if records:
        kernels = kernel_table(records)
        agg = {}
        for name, e0, e1, work in records:
            a = agg.setdefault(name, [0, 0.0, 0])
            a[0] += 1
            a[1] += e0.elapsed_time(e1)
            a[2] += work
        n, ms, work = agg["gemm_nt"]
        achieved = work / (ms * 1e-3) / 1e12
        picked = {ops.gemm_pick(*mnk) for mnk in ((TOKENS, FFN, DIM), (TOKENS, DIM, FFN), (FFN, DIM, TOKENS))}
        if args.algo:
            picked = {(args.algo, ops.gemm_algos()[args.algo - 1])}
        traffic, traffic_kernel = gemm_traffic_bytes()
        names = sorted(name for _, name in picked)
        roofline = {"kernel": " / ".join(names) + " (fp8 e4m3 NT GEMM, 2*16384*4096*11008 flop per launch; forward, dgrad and wgrad products)",
                    "bound": "mfma", "achieved": round(achieved, 1), "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                    "frac": round(achieved / PEAK_FP8_TFLOPS, 4),
                    # counters of another tile configuration say nothing about this one
                    "traffic": traffic if names == [traffic_kernel] else None,
                    "traffic_unit": "bytes per launch, mean of the step's three products (algorithmic: 390 MB); from "
                                    "profiles/gemm_nt_7b_hbm_traffic.txt (rocprofv3 FETCH_SIZE / WRITE_SIZE runs of "
                                    + traffic_kernel + ")"}

    out = {
        "metric": "fp8 rowwise linear fwd+bwd TFLOP/s at 7B MLP",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn",
        "data": "synthetic",
        "config": {"workload": "llama-7B SwiGLU MLP fwd+bwd, row-wise fp8 (configs[2])", "dim": DIM, "ffn": FFN,
                   "tokens": TOKENS, "flop_per_step": STEP_FLOP, "gemm_algo": args.algo,
                   "wgrad": "fp8", "scale_rule": ops.get_scale_rule()},
        "frac_of_fp8_peak": round(tflops / PEAK_FP8_TFLOPS, 4),
        "roofline": roofline,
        "kernels": kernels,
    }
    if not args.no_extras:
        out["sustained"] = sustained(mlp, args.sustained_seconds)
        out["extras"] = extras(torch, mlp, timed, args)
        del mlp, model, x, gy
        torch.cuda.empty_cache()
        out["extras"].update(more_extras(torch, dev, args))
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch, args.cpu_sample_tokens)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
