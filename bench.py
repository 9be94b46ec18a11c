#!/usr/bin/env python3
"""Benchmark of the Quartet MXFP4 linear hot path on one MI355X.

A "step" is one forward + backward of one Quartet-quantized linear layer (quest-RTN forward,
absmax stochastic-rounding backward with sign re-randomisation, Hadamard block 32) on the
isolated 7B-class shape: tokens 8192, in 4096, out 4096, bf16 inputs resident in HBM.
Prints ONE JSON line; `value` = 6*T*I*O / step time in TFLOP/s.  The line also carries the
roofline of the dominant kernel (the FP4 GEMM, MFMA-bound), the HBM roofline of the
Hadamard+quantize kernel, per-kernel timings, and a CPU baseline (the CPU restatement of the same
pseudo-quantized linear timed on this host on a bounded row sample)."""
import argparse
import json
import os
import sys
import time

import torch

T_TOKENS, IN_F, OUT_F = 8192, 4096, 4096
PEAK_FP4_TFLOPS = 10100.0   # MI355X dense MXFP4 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
# HBM bytes per launch from profiler byte counters (fetch + write), scaled by what the same counters read for a
# plain 256 MiB device copy (fetch counter x 2.0 KiB, write counter x 1.0 KiB)
GEMM_TRAFFIC_BYTES = 173.9e6      # mean of the three GEMMs: 108.7 MiB fetched (operand re-reads that miss L2) + 57.1 MiB written
QUANTIZE_TRAFFIC_BYTES = 90.3e6   # two thirds (the X share) of the forward pair launch: 96.1 MiB fetched + 33.0 MiB written; algorithmic 89.1e6


def make_inputs(device, tokens=T_TOKENS, seed=0):
    """X ~ N(0,1) with 1% Student-t(3) entries, W ~ N(0, 0.02), dY ~ N(0, 1e-3); generated on the CPU
    with a seeded generator so the CPU baseline and the GPU see identical bits."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(tokens, IN_F, generator=g)
    heavy = torch.rand(tokens, IN_F, generator=g) < 0.01
    chi2 = (torch.randn(3, tokens, IN_F, generator=g) ** 2).sum(0)
    x = torch.where(heavy, torch.randn(tokens, IN_F, generator=g) / torch.sqrt(chi2 / 3.0), x)
    w = 0.02 * torch.randn(OUT_F, IN_F, generator=g)
    dy = 1e-3 * torch.randn(tokens, OUT_F, generator=g)
    return x.to(torch.bfloat16).to(device), w.to(torch.bfloat16).to(device), dy.to(torch.bfloat16).to(device)


def build_layer(device):
    import quartet_amd as q
    layer = q.QuantizedLinear(
        IN_F, OUT_F, bias=False,
        weight_quantizer=q.QUANTIZER_CLASSES["QuestMXFP4Quantizer"](hadamard_dim=32),
        activation_quantizer=q.QUANTIZER_CLASSES["QuestMXFP4Quantizer"](hadamard_dim=32),
        gradient_quantizer=q.QUANTIZER_CLASSES["AlbertTsengQuantizer"](hadamard_dim=32, stochastic=True, rerotate="signs"),
        backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"](),
    ).to(device=device, dtype=torch.bfloat16)
    return layer


def time_kernel(fn, reps=20, warmup=3, graph=True):
    """Average duration (ms) of one launch sequence `fn`, HIP events on the stream the kernels run on.

    With `graph` the `reps` launches are recorded into one HIP graph and the replay is timed: the kernels then follow
    each other as closely as the hardware dispatches them, so a 10-20 us kernel is not measured through the host's
    launch rate (Python + allocator + ctypes cost about as much per call as such a kernel runs)."""
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    if graph:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(reps):
                fn()
        g.replay()
        torch.cuda.synchronize()
        start.record()
        g.replay()
        stop.record()
        stop.synchronize()
        ms = start.elapsed_time(stop) / reps
        del g
        return ms
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


COLD_CYCLE_BYTES = 1 << 30  # distinct input bytes walked before a buffer repeats: 4x the 256 MB memory-side cache


def time_kernel_cold(make_call, inputs, reps=24, warmup=2):
    """HBM-cold timing: `inputs` are the tensors one launch reads; the launch is timed over clones of them that
    together exceed the last-level cache several times, so every launch streams its input from HBM."""
    nbytes = sum(t.numel() * t.element_size() for t in inputs)
    n = max(2, min(64, -(-COLD_CYCLE_BYTES // max(nbytes, 1))))
    sets = [inputs] + [[t.clone() for t in inputs] for _ in range(n - 1)]
    calls = [make_call(*st) for st in sets]
    state = {"i": 0}

    def fn():
        calls[state["i"] % n]()
        state["i"] += 1
    return time_kernel(fn, reps=max(reps, n), warmup=warmup)


def kernel_breakdown(x, w, dy):
    """Per-kernel timings of the eleven launches of one step, with algorithmic bytes / flops.  HBM-bound kernels
    are timed HBM-cold (see time_kernel_cold) and, for reference, warm on one buffer."""
    from quartet_amd import kernels as K
    T, I, O = x.shape[0], x.shape[1], w.shape[0]
    out = {}
    tl = True  # tiled code bytes, as the layer uses for these extents
    xc, xs, xm, _ = K.quantize_mxfp4(x, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)
    wc, ws, wm, _ = K.quantize_mxfp4(w, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)
    signs = 0x5A5AA5A5
    ec, es, _, _ = K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, seed=1, tiled=tl)
    etc, ets, _, _ = K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, transposed_in=True, seed=2, tiled=tl)
    wtc, wts, _ = K.requantize_transposed_mxfp4(wc, ws, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=3, tiled_in=tl, tiled_out=tl)
    xtc, xts, _ = K.requantize_transposed_mxfp4(xc, xs, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=4, tiled_in=tl, tiled_out=tl)
    gxq = K.gemm_mxfp4_tn(ec, es, wtc, wts, 1.0, torch.bfloat16, a_tiled=tl, b_tiled=tl)
    gwq = K.gemm_mxfp4_tn(etc, ets, xtc, xts, 1.0, torch.bfloat16, a_tiled=tl, b_tiled=tl)

    def hbm(name, elems, bytes_per_elem, make_call, inputs):
        cold = time_kernel_cold(make_call, inputs)
        warm = time_kernel(make_call(*inputs))
        out[name] = {"ms": round(cold, 4), "GBps": round(elems * bytes_per_elem / cold / 1e6, 1),
                     "bytes_per_elem": bytes_per_elem, "ms_warm": round(warm, 4)}

    def mfma(name, m, n, k, fn):
        ms = time_kernel(fn)
        out[name] = {"ms": round(ms, 4), "TFLOPs": round(2.0 * m * n * k / ms / 1e9, 1), "shape": [m, n, k]}

    hbm("quantize_x_quest_rtn_mask", T * I, 2.65625,
        lambda a: (lambda: K.quantize_mxfp4(a, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)), [x])
    hbm("quantize_w_quest_rtn_mask", O * I, 2.65625,
        lambda a: (lambda: K.quantize_mxfp4(a, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)), [w])
    mfma("gemm_fwd", T, O, I, lambda: K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.bfloat16, a_tiled=tl, b_tiled=tl))
    hbm("quantize_e_absmax_sr", T * O, 2.53125,
        lambda a: (lambda: K.quantize_mxfp4(a, 32, signs, K.QM_ABSMAX_SR, seed=1, tiled=tl)), [dy])
    hbm("quantize_et_absmax_sr_transposed", T * O, 2.53125,
        lambda a: (lambda: K.quantize_mxfp4(a, 32, signs, K.QM_ABSMAX_SR, transposed_in=True, seed=2, tiled=tl)), [dy])
    hbm("requantize_wt", O * I, 1.0625,
        lambda c, sc: (lambda: K.requantize_transposed_mxfp4(c, sc, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=3,
                                                              tiled_in=tl, tiled_out=tl)),
        [wc, ws])
    hbm("requantize_xt", T * I, 1.0625,
        lambda c, sc: (lambda: K.requantize_transposed_mxfp4(c, sc, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=4,
                                                              tiled_in=tl, tiled_out=tl)),
        [xc, xs])
    mfma("gemm_dgrad", T, I, O, lambda: K.gemm_mxfp4_tn(ec, es, wtc, wts, 1.0, torch.bfloat16, a_tiled=tl, b_tiled=tl))
    mfma("gemm_wgrad", O, I, T, lambda: K.gemm_mxfp4_tn(etc, ets, xtc, xts, 1.0, torch.bfloat16, a_tiled=tl, b_tiled=tl))
    hbm("hadamard_bwd_x", T * I, 4.125,
        lambda g, m: (lambda: K.masked_hadamard_bwd(g, 32, torch.bfloat16, None, m)), [gxq, xm])
    hbm("hadamard_bwd_w", O * I, 4.125,
        lambda g, m: (lambda: K.masked_hadamard_bwd(g, 32, torch.bfloat16, None, m)), [gwq, wm])
    return out


def quantizer_sweep(device):
    """Quantizer-only throughput (HBM-cold) on [rows x 4096] bf16 with 0.1 % entries at +-1e3, for the three
    production modes and Hadamard blocks 32/64/128."""
    from quartet_amd import kernels as K
    res = []
    for rows in (4096, 16384, 65536):
        g = torch.Generator().manual_seed(rows)
        x = torch.randn(rows, 4096, generator=g)
        spike = torch.rand(rows, 4096, generator=g) < 1e-3
        sgn = torch.where(torch.rand(rows, 4096, generator=g) < 0.5, -1e3, 1e3)
        x = torch.where(spike, sgn, x).to(torch.bfloat16).to(device)
        for hd in (32, 64, 128):
            for name, mode, mask, bpe in (("quest_rtn_mask", K.QM_QUEST_RTN, True, 2.65625),
                                          ("absmax_rtn", K.QM_ABSMAX_RTN, False, 2.53125),
                                          ("absmax_sr", K.QM_ABSMAX_SR, False, 2.53125)):
                ms = time_kernel_cold(lambda a: (lambda: K.quantize_mxfp4(a, hd, None, mode, want_mask=mask, seed=7)), [x],
                                      reps=8, warmup=1)
                res.append({"rows": rows, "hd": hd, "mode": name, "ms": round(ms, 4),
                            "GBps": round(rows * 4096 * bpe / ms / 1e6, 1)})
    res.append(cpu_quantizer_baseline())
    return res


def cpu_quantizer_baseline(rows=4096):
    """The CPU oracle's quantizer on [rows x 4096] bf16 (quest RTN + mask, Hadamard 32): one thread, and all host threads."""
    import ctypes

    from oracle import oracle as o
    from tests.util import to_oracle
    x = to_oracle(torch.randn(rows, 4096, generator=torch.Generator().manual_seed(0)).to(torch.bfloat16))
    o.lib()
    gomp = ctypes.CDLL("libgomp.so.1")
    out = {"cpu_oracle_quantizer": f"[{rows} x 4096] bf16, quest RTN + mask, hd 32; 2.65625 B/elt"}
    for label, n in (("one_thread", 1), ("all_threads", min(os.cpu_count() or 1, 16))):
        gomp.omp_set_num_threads(n)
        o.quantize(x[:64], 32, mode=o.QUEST_RTN, want_mask=True)
        t0 = time.perf_counter()
        o.quantize(x, 32, mode=o.QUEST_RTN, want_mask=True)
        dt = time.perf_counter() - t0
        out[label] = {"threads": n, "GBps": round(rows * 4096 * 2.65625 / dt / 1e9, 3)}
    return out


def _cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(sample_tokens=T_TOKENS):
    """The CPU restatement of the same pseudo-quantized linear (oracle quantizers + fp32 BLAS matmuls on
    de-quantized operands, i.e. the op sequence the reference runs) on a row sample of the workload."""
    import numpy as np
    from oracle import oracle as o
    from tests.util import to_oracle
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    x, w, dy = make_inputs("cpu", tokens=sample_tokens)
    xo, wo, eo = to_oracle(x), to_oracle(w), to_oracle(dy)
    o.lib()
    d = float(o.FOUR_THIRDS)
    signs = np.where(np.arange(32) % 3 == 0, -1, 1)

    def deq(q, post=1.0):
        return torch.from_numpy(o.dequantize(q["codes"], q["scales"], post))

    def one_pass():
        t0 = time.perf_counter()
        qx = o.quantize(xo, 32, mode=o.QUEST_RTN, want_mask=True)
        qw = o.quantize(wo, 32, mode=o.QUEST_RTN, want_mask=True)
        y = deq(qx) @ deq(qw).T
        qe = o.quantize(eo, 32, signs=signs, mode=o.ABSMAX_SR, seed=1)
        qwt = o.requantize_transposed(qw["codes"], qw["scales"], hd=32, signs=signs, mode=o.ABSMAX_SR, seed=2)
        gxq = deq(qe, d) @ deq(qwt, d).T
        qet = o.quantize(eo, 32, signs=signs, mode=o.ABSMAX_SR, transposed_in=True, seed=3)
        qxt = o.requantize_transposed(qx["codes"], qx["scales"], hd=32, signs=signs, mode=o.ABSMAX_SR, seed=4)
        gwq = deq(qet, d) @ deq(qxt, d).T
        gx = o.masked_hadamard_bwd(gxq.numpy(), 32, o.BF16, None, qx["mask"])
        gw = o.masked_hadamard_bwd(gwq.numpy(), 32, o.BF16, None, qw["mask"])
        return time.perf_counter() - t0, y, gx, gw
    times = []
    for _ in range(3):  # median of three passes over the whole workload
        dt, y, gx, gw = one_pass()
        times.append(dt)
    dt = sorted(times)[1]
    assert y.shape[0] == sample_tokens and gx.shape == (sample_tokens, IN_F) and gw.shape == (OUT_F, IN_F)
    flops = 6.0 * sample_tokens * IN_F * OUT_F
    return {"value": round(flops / dt / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"fwd+bwd on {sample_tokens} of {T_TOKENS} tokens (same I={IN_F}, O={OUT_F}), median of 3 passes; "
                      f"CPU oracle quantizers + fp32 BLAS matmuls on de-quantized operands, {dt:.2f} s per pass",
            "cpu_model": _cpu_model()}


def library_gemm(device, reps=50):
    """The vendor library's block-scaled FP4 product (hipBLASLt behind torch._scaled_mm) on the forward GEMM's shape and
    operand formats, for context next to the hand-written kernel: random codes, unit scales."""
    M, N, K = T_TOKENS, OUT_F, IN_F
    try:
        a = torch.randint(0, 256, (M, K // 2), dtype=torch.uint8, device=device).view(torch.float4_e2m1fn_x2)
        b = torch.randint(0, 256, (N, K // 2), dtype=torch.uint8, device=device).view(torch.float4_e2m1fn_x2)
        sa = torch.full((M, K // 32), 127, dtype=torch.uint8, device=device).view(torch.float8_e8m0fnu)
        sb = torch.full((N, K // 32), 127, dtype=torch.uint8, device=device).view(torch.float8_e8m0fnu)
        run = lambda: torch._scaled_mm(a, b.t(), sa, sb, out_dtype=torch.bfloat16)
        ms = time_kernel(run, reps=reps, warmup=5, graph=False)
    except Exception as exc:  # the installed torch / hipBLASLt may not offer this product
        return {"error": f"{type(exc).__name__}: {str(exc)[:200]}"}
    return {"what": f"torch._scaled_mm float4_e2m1fn_x2 x float4_e2m1fn_x2, e8m0 scales per 32, {M}x{N}x{K}, bf16 out",
            "ms": round(ms, 4), "TFLOPs": round(2.0 * M * N * K / ms / 1e9, 1)}


def gemm_operand_content(x, w, dy, rounds=3):
    """The forward product's shape timed on operands of different content.  The kernel is power-limited: the clock the
    chip holds, and with it the duration, follows how much the operand bits toggle, so constant operands show what the
    kernel's structure alone costs."""
    from quartet_amd import kernels as K
    signs = 0x5A5AA5A5
    xc, xs, _, _ = K.quantize_mxfp4(x, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=True)
    wc, ws, _, _ = K.quantize_mxfp4(w, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=True)
    ec, es, _, _ = K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, seed=1, tiled=True)
    wtc, wts, _ = K.requantize_transposed_mxfp4(wc, ws, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=3, tiled_in=True,
                                                tiled_out=True)
    rand = lambda t: torch.randint(0, 256, t.shape, dtype=torch.uint8, device=t.device)
    cases = [("quest_rtn_codes_of_gaussians", xc, xs, wc, ws), ("absmax_sr_codes_of_gaussians", ec, es, wtc, wts),
             ("uniform_random_codes", rand(xc), xs, rand(wc), ws), ("all_zero_codes", torch.zeros_like(xc), xs, torch.zeros_like(wc), ws),
             ("constant_codes_1.0", torch.full_like(xc, 0x22), xs, torch.full_like(wc, 0x22), ws)]
    out = {}
    for _ in range(rounds):  # interleaved rounds: the box's clock drifts over seconds
        for name, a, sa, b, sb in cases:
            ms = time_kernel(lambda: K.gemm_mxfp4_tn(a, sa, b, sb, 1.0, torch.bfloat16, a_tiled=True, b_tiled=True), reps=30)
            out.setdefault(name, []).append(ms)
    flops = 2.0 * T_TOKENS * IN_F * OUT_F
    return {k: {"ms": round(sorted(v)[len(v) // 2], 4), "TFLOPs": round(flops / sorted(v)[len(v) // 2] / 1e9, 1)} for k, v in out.items()}


def llama_step(args, device):
    """Whole-model step of a Llama configuration with every block linear on the Quartet path: bf16 autocast around
    forward and backward, cross-entropy on random ids, AdamW (fp32 state) for the ~800 M configuration."""
    from quartet_amd import llama as L
    torch.manual_seed(0)
    over = L.unquantized() if args.unquantized else {}
    over["sdpa_backend"] = args.sdpa
    if args.workload == "llama30m":
        cfg, batch, seq, opt_step = L.llama_30m(**over), 64, 512, False
    else:
        cfg, batch, seq, opt_step = L.llama_800m(**over), 16, 2048, True
    model = L.Llama(cfg).to(device)
    opt = torch.optim.AdamW(model.parameters(), lr=1e-4, fused=True) if opt_step else None
    g = torch.Generator().manual_seed(1)
    idx = torch.randint(0, cfg.vocab_size, (batch, seq), generator=g).to(device)
    tgt = torch.randint(0, cfg.vocab_size, (batch, seq), generator=g).to(device)

    def step():
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            loss = model(idx, targets=tgt)["loss"]
            loss.backward()
        if opt is not None:
            opt.step()
        model.zero_grad(set_to_none=True)
        return loss

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / args.steps * 1e3
    peak_gib = torch.cuda.max_memory_allocated() / 2 ** 30
    lin = sum(m.weight.numel() for _, m in model.block_linears())
    tokens = batch * seq
    flops = 6.0 * tokens * lin
    return {"metric": "Quartet linear fwd+bwd TFLOPS (MXFP4 MFMA) + Hadamard/quantize HBM GB/s",
            "value": round(flops / (ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": round(ms, 3), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16" if args.unquantized else "mxfp4", "data": "synthetic",
            "config": {"workload": f"{args.workload}{' (unquantized bf16 linears)' if args.unquantized else ''} whole-model step ({cfg.n_layer} layers, d {cfg.n_embd}, {batch}x{seq} tokens, "
                                   f"{'fwd+bwd+AdamW' if opt_step else 'fwd+bwd'}); value counts the block linears' 6*tokens*params "
                                   f"flops only ({flops / 1e12:.2f} TFLOP) over the whole step time"},
            "tokens_per_s": round(tokens / (ms * 1e-3), 1), "final_loss": round(float(loss.detach()), 4),
            "peak_allocated_GiB": round(peak_gib, 2)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-breakdown", action="store_true")
    ap.add_argument("--workload", default="linear", choices=["linear", "llama30m", "llama800m"],
                    help="linear (default): the isolated 8192x4096x4096 layer the metric is quoted on; llama30m / llama800m: "
                         "whole-model fwd+bwd(+AdamW) step of the 30 M / ~800 M Llama configurations, reported in the same unit "
                         "over the block linears' flops")
    ap.add_argument("--unquantized", action="store_true",
                    help="with a llama workload: identity quantizers and the plain scheme (the bf16 model, for context)")
    ap.add_argument("--sdpa", default="auto", choices=["auto", "default"],
                    help="llama workloads: library attention kernels tried in the model's own order (auto) or the dispatcher's (default)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a known-traffic kernel for scaling profiler byte counters)")
    ap.add_argument("--quantizer-sweep", action="store_true",
                    help="also time the quantizer alone on [rows x 4096] for rows 4096/16384/65536, three modes, hd 32/64/128")
    ap.add_argument("--gemm-operand-content", action="store_true",
                    help="also time the forward GEMM on operands of different content (real codes, random, constant): shows the power limit")
    ap.add_argument("--library-gemm", action="store_true",
                    help="also time the vendor library's MXFP4 product (torch._scaled_mm) on the forward GEMM's shape, for context")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the quantized-linear path has no CPU fallback")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    device = torch.device("cuda:0")
    if args.workload != "linear":
        print(json.dumps(llama_step(args, device)))
        return
    x, w, dy = make_inputs(device)
    layer = build_layer(device)
    with torch.no_grad():
        layer.weight.copy_(w)
    x.requires_grad_(True)

    def step():
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            y = layer(x)
        y.backward(dy)
        x.grad = None
        layer.weight.grad = None

    if args.calibration_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    flops = 6.0 * T_TOKENS * IN_F * OUT_F
    result = {
        "metric": "Quartet linear fwd+bwd TFLOPS (MXFP4 MFMA) + Hadamard/quantize HBM GB/s",
        "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "mxfp4", "data": "synthetic",
        "config": {"workload": "isolated Quartet linear fwd+dgrad+wgrad, tokens 8192 x in 4096 x out 4096, "
                               "bf16 X/W/dY, quest-RTN forward, absmax-SR backward, Hadamard 32"},
    }
    if not args.no_breakdown:
        x.requires_grad_(False)
        kb = kernel_breakdown(x.detach(), w, dy)
        result["kernels"] = kb
        # the three GEMMs of a step (fwd, dgrad, wgrad) run the same kernel on the same flop count: the roofline
        # entry is their mean, which is what a profiler's per-kernel average over the run reports
        gemms = [kb[k] for k in ("gemm_fwd", "gemm_dgrad", "gemm_wgrad")]
        gemm_ms = sum(g["ms"] for g in gemms) / 3.0
        gemm_tf = 2.0 * T_TOKENS * IN_F * OUT_F / gemm_ms / 1e9
        result["roofline"] = {"bound": "mfma", "kernel": "gemm_mxfp4_tn_big4_kernel (8192x4096x4096, 8192x4096x4096, 4096x4096x8192)",
                              "achieved": round(gemm_tf, 1), "peak": PEAK_FP4_TFLOPS, "unit": "TFLOP/s",
                              "frac": round(gemm_tf / PEAK_FP4_TFLOPS, 4), "traffic": GEMM_TRAFFIC_BYTES,
                              "avg_launch_ms": round(gemm_ms, 4)}
        qk = kb["quantize_x_quest_rtn_mask"]
        result["roofline_quantize"] = {"bound": "hbm", "kernel": "quantize_rowmajor (quest RTN + mask, 8192x4096 bf16)",
                                       "achieved": qk["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                       "frac": round(qk["GBps"] / PEAK_HBM_GBS, 4), "traffic": QUANTIZE_TRAFFIC_BYTES,
                                       "avg_launch_ms": qk["ms"]}
    if args.quantizer_sweep:
        result["quantizer_sweep"] = quantizer_sweep(device)
    if args.library_gemm:
        result["library_gemm"] = library_gemm(device)
    if args.gemm_operand_content:
        result["gemm_operand_content"] = gemm_operand_content(x.detach(), w, dy)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
