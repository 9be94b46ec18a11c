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

T_TOKENS, IN_F, OUT_F = 8192, 4096, 4096   # OUT_F: default of --out-features (the configuration's other value is 11008)
PEAK_FP4_TFLOPS = 10100.0   # MI355X dense MXFP4 MFMA
PEAK_HBM_GBS = 8000.0       # MI355X HBM3E
ROOT = os.path.dirname(os.path.abspath(__file__))
# HBM bytes per launch come from profiler byte counters (two rocprofv3 --pmc runs of this script, FETCH_SIZE then
# WRITE_SIZE, scaled by what the same counters read for a plain 256 MiB device copy).  `--counters-to-json` turns the
# two runs' CSV files into this tracked file, which also records the commit and a hash of the kernel sources it was
# taken at; the roofline entries quote it together with whether it still matches the sources of this build.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")


def make_inputs(device, tokens=T_TOKENS, seed=0, out_f=OUT_F):
    """X ~ N(0,1) with 1% Student-t(3) entries, W ~ N(0, 0.02), dY ~ N(0, 1e-3); generated on the CPU
    with a seeded generator so the CPU baseline and the GPU see identical bits."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(tokens, IN_F, generator=g)
    heavy = torch.rand(tokens, IN_F, generator=g) < 0.01
    chi2 = (torch.randn(3, tokens, IN_F, generator=g) ** 2).sum(0)
    x = torch.where(heavy, torch.randn(tokens, IN_F, generator=g) / torch.sqrt(chi2 / 3.0), x)
    w = 0.02 * torch.randn(out_f, IN_F, generator=g)
    dy = 1e-3 * torch.randn(tokens, out_f, generator=g)
    return x.to(torch.bfloat16).to(device), w.to(torch.bfloat16).to(device), dy.to(torch.bfloat16).to(device)


def build_layer(device, out_f=OUT_F):
    import quartet_amd as q
    layer = q.QuantizedLinear(
        IN_F, out_f, bias=False,
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


def kernel_breakdown(x, w, dy, only_gemms=False):
    """Per-kernel timings of the launches of one step, with algorithmic bytes / flops ("in_step": false marks a kernel
    the step does not run at this shape, timed for comparison).  HBM-bound kernels are timed HBM-cold (see
    time_kernel_cold) and, for reference, warm on one buffer."""
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
    d2 = K.FOUR_THIRDS ** 2
    # the two gradient products as the layer step runs them at this shape: the masked inverse rotation (B7 / B8) in the epilogue
    fused = K.gemm_fuses_rotation(es, wts, T, I, O) and K.gemm_fuses_rotation(ets, xts, O, I, T)

    def dgrad():
        return (K.gemm_mxfp4_tn_rotated(ec, es, wtc, wts, xm, d2, torch.bfloat16, None, a_tiled=tl, b_tiled=tl) if fused
                else K.gemm_mxfp4_tn(ec, es, wtc, wts, d2, torch.bfloat16, a_tiled=tl, b_tiled=tl))

    def wgrad():
        return (K.gemm_mxfp4_tn_rotated(etc, ets, xtc, xts, wm, d2, torch.bfloat16, None, a_tiled=tl, b_tiled=tl) if fused
                else K.gemm_mxfp4_tn(etc, ets, xtc, xts, d2, torch.bfloat16, a_tiled=tl, b_tiled=tl))

    def hbm(name, elems, bytes_per_elem, make_call, inputs):
        cold = time_kernel_cold(make_call, inputs)
        warm = time_kernel(make_call(*inputs))
        out[name] = {"ms": round(cold, 4), "GBps": round(elems * bytes_per_elem / cold / 1e6, 1),
                     "bytes_per_elem": bytes_per_elem, "ms_warm": round(warm, 4)}

    def mfma(name, m, n, k, fn):
        ms = time_kernel(fn)
        out[name] = {"ms": round(ms, 4), "TFLOPs": round(2.0 * m * n * k / ms / 1e9, 1), "shape": [m, n, k]}

    def products():
        mfma("gemm_fwd", T, O, I, lambda: K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.bfloat16, a_tiled=tl, b_tiled=tl))
        mfma("gemm_dgrad", T, I, O, dgrad)
        mfma("gemm_wgrad", O, I, T, wgrad)
        if fused:
            for k in ("gemm_dgrad", "gemm_wgrad"):
                out[k]["epilogue"] = "masked inverse rotation (hadamard_bwd) fused"
            mfma("gemm_dgrad_plain", T, I, O, lambda: K.gemm_mxfp4_tn(ec, es, wtc, wts, d2, torch.bfloat16, a_tiled=tl, b_tiled=tl))
            mfma("gemm_wgrad_plain", O, I, T, lambda: K.gemm_mxfp4_tn(etc, ets, xtc, xts, d2, torch.bfloat16, a_tiled=tl, b_tiled=tl))
            for k in ("gemm_dgrad_plain", "gemm_wgrad_plain"):
                out[k]["in_step"] = False

    if only_gemms:
        products()
        return out
    hbm("quantize_x_quest_rtn_mask", T * I, 2.65625,
        lambda a: (lambda: K.quantize_mxfp4(a, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)), [x])
    hbm("quantize_w_quest_rtn_mask", O * I, 2.65625,
        lambda a: (lambda: K.quantize_mxfp4(a, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)), [w])
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
    products()
    # the stand-alone inverse rotation: in the step only where the products' epilogue does not carry it
    hbm("hadamard_bwd_x", T * I, 4.125,
        lambda g, m: (lambda: K.masked_hadamard_bwd(g, 32, torch.bfloat16, None, m)), [gxq, xm])
    hbm("hadamard_bwd_w", O * I, 4.125,
        lambda g, m: (lambda: K.masked_hadamard_bwd(g, 32, torch.bfloat16, None, m)), [gwq, wm])
    for k in ("hadamard_bwd_x", "hadamard_bwd_w"):
        out[k]["in_step"] = not fused
    return out


def in_step_gemm_ms_by_difference(x, w, dy, fused, steps=10, rounds=5):
    """Mean duration of the three products inside the layer step, from two HIP graphs timed with events: the step's
    kernels launched one by one in the layer's order (`steps` times), and the same sequence without the three
    products.  The difference of the two replays is what the step pays for its products where they actually run --
    between quantizer kernels -- with no event or host time inside the measured interval.  `fused`: the two gradient
    products carry the masked inverse rotation in their epilogue, as the layer runs them where the kernel serves the
    shape (the step then has no inverse-rotation kernels); otherwise plain products and the two rotation kernels."""
    from quartet_amd import kernels as K
    tl, signs = True, 0x5A5AA5A5

    def one_step(full):
        def product(ac, as_, bc, bs, alpha, mask=None):
            if not full:
                return None
            if mask is not None and fused:
                return K.gemm_mxfp4_tn_rotated(ac, as_, bc, bs, mask, alpha, torch.bfloat16, None, a_tiled=tl, b_tiled=tl)
            return K.gemm_mxfp4_tn(ac, as_, bc, bs, alpha, torch.bfloat16, a_tiled=tl, b_tiled=tl)
        xc, xs, xm, _ = K.quantize_mxfp4(x, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)
        wc, ws, wm, _ = K.quantize_mxfp4(w, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)
        product(xc, xs, wc, ws, 1.0)
        ec, es, _, _ = K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, seed=1, tiled=tl)
        etc, ets, _, _ = K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, transposed_in=True, seed=2, tiled=tl)
        wtc, wts, _ = K.requantize_transposed_mxfp4(wc, ws, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=3, tiled_in=tl, tiled_out=tl)
        xtc, xts, _ = K.requantize_transposed_mxfp4(xc, xs, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=4, tiled_in=tl, tiled_out=tl)
        gxq = product(ec, es, wtc, wts, K.FOUR_THIRDS ** 2, xm)
        gwq = product(etc, ets, xtc, xts, K.FOUR_THIRDS ** 2, wm)
        if not fused:
            K.masked_hadamard_bwd(gxq if full else x, 32, torch.bfloat16, None, xm)
            K.masked_hadamard_bwd(gwq if full else w, 32, torch.bfloat16, None, wm)

    graphs = {}
    for full in (True, False):
        one_step(full)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(steps):
                one_step(full)
        g.replay()
        graphs[full] = g
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    times = {True: [], False: []}
    for _ in range(rounds):
        for full in (True, False):
            torch.cuda.synchronize()
            start.record()
            graphs[full].replay()
            stop.record()
            stop.synchronize()
            times[full].append(start.elapsed_time(stop) / steps)
    med = {k: sorted(v)[len(v) // 2] for k, v in times.items()}
    return {"ms": (med[True] - med[False]) / 3.0, "step_graph_ms": round(med[True], 4), "step_graph_without_products_ms": round(med[False], 4)}


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


def cpu_baseline(sample_tokens=T_TOKENS, out_f=OUT_F):
    """The CPU restatement of the same pseudo-quantized linear (oracle quantizers + fp32 BLAS matmuls on
    de-quantized operands, i.e. the op sequence the reference runs) on a row sample of the workload."""
    import numpy as np
    from oracle import oracle as o
    from tests.util import to_oracle
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    x, w, dy = make_inputs("cpu", tokens=sample_tokens, out_f=out_f)
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
    assert y.shape[0] == sample_tokens and gx.shape == (sample_tokens, IN_F) and gw.shape == (out_f, IN_F)
    flops = 6.0 * sample_tokens * IN_F * out_f
    return {"value": round(flops / dt / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"fwd+bwd on {sample_tokens} of {T_TOKENS} tokens (same I={IN_F}, O={out_f}), median of 3 passes; "
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


def gemm_tile_phases(x, w, launches=5):
    """Where a tile's time goes in the forward product: the persistent kernel's stamping instantiation records the shader
    clock around every tile's K loop and epilogue (thread 0 of each workgroup).  No matrix instruction runs during an
    epilogue, so its share of a tile is the share of the launch the matrix pipe idles for at the tile boundaries."""
    import statistics
    from quartet_amd import kernels as K
    xc, xs, _, _ = K.quantize_mxfp4(x, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=True)
    wc, ws, _, _ = K.quantize_mxfp4(w, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=True)
    for _ in range(40):   # the state the chip is in during the step: clocks settled under this kernel
        K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.bfloat16, a_tiled=True, b_tiled=True)
    ksteps = x.shape[1] // 128

    def stamps(maskbits):
        k_loop, epi, span = [], [], []
        for _ in range(launches):
            _, st = K.gemm_tile_phases(xc, xs, wc, ws, 1.0, a_tiled=True, b_tiled=True, maskbits=maskbits)
            st = st.tolist()
            for row in st:
                start = row[1]
                for i in range(2, len(row) - 1, 2):
                    if row[i] == 0:
                        break
                    k_loop.append(row[i] - start)
                    epi.append(row[i + 1] - row[i])
                    start = row[i + 1]
            span.append(max(max(r) - r[0] for r in st))   # per workgroup: the XCDs' counters are not aligned with each other
        return k_loop, epi, span, st

    k_loop, epi, span, st = stamps(None)
    kl, ep = statistics.median(k_loop), statistics.median(epi)
    # the same launch with the masked inverse rotation in the epilogue (as the step's two gradient products run), on a mask
    # of the output's shape
    rot = {}
    if K.gemm_fuses_rotation(xs, ws, x.shape[0], w.shape[0], x.shape[1]):
        g = torch.Generator(device=x.device).manual_seed(3)
        keep = torch.randint(0, 256, (x.shape[0], w.shape[0] // 8), generator=g, dtype=torch.uint8, device=x.device)
        rk, re_, rs, _ = stamps(keep)
        rot = {"with_inverse_rotation": {"cycles_per_k_step": round(statistics.median(rk) / ksteps, 1), "epilogue_cycles": int(statistics.median(re_)),
                                         "longest_workgroup_cycles": int(statistics.median(rs))}}
    return {"what": "shader-clock stamps of the forward product's kernel, medians over every tile of %d launches" % launches, **rot,
            "tiles_per_workgroup": len(k_loop) // max(1, launches * len(st)),
            "k_loop_cycles": int(kl), "cycles_per_k_step": round(kl / ksteps, 1), "epilogue_cycles": int(ep),
            "epilogue_share_of_tile": round(ep / (kl + ep), 4),
            "k_loop_matrix_pipe_duty": round(32 * 32 * ksteps / kl, 4),   # 32 instructions of 32 cycles per K step per SIMD
            "longest_workgroup_cycles": int(statistics.median(span)),
            "matrix_pipe_duty_of_the_launch": round(32 * 32 * ksteps * (len(k_loop) / max(1, launches * len(st))) / statistics.median(span), 4)}


def mfma_only_ceiling(x, w, iters=400, rounds=3):
    """The FP4 matrix instruction alone (no loads, no epilogue) on the bytes of the forward product's real operands, on
    uniformly random bytes and on zero bytes: what the chip sustains for this instruction at its power limit, which is
    the ceiling the product's own rate is to be read against."""
    from quartet_amd import kernels as K
    xc, _, _, _ = K.quantize_mxfp4(x, 32, None, K.QM_QUEST_RTN, tiled=True)
    wc, _, _, _ = K.quantize_mxfp4(w, 32, None, K.QM_QUEST_RTN, tiled=True)
    real = torch.cat([xc.flatten()[: 8 << 20], wc.flatten()[: 8 << 20]]).contiguous()
    cases = {"quest_rtn_codes_of_the_forward_operands": real,
             "uniform_random_bytes": torch.randint(0, 256, (16 << 20,), dtype=torch.uint8, device=x.device),
             "zero_bytes": torch.zeros(16 << 20, dtype=torch.uint8, device=x.device)}
    out = {}
    for _ in range(rounds):
        for name, buf in cases.items():
            n = [0]

            def run():
                n[0] = K.mfma_only(buf, iters)
            ms = time_kernel(run, reps=10, warmup=2, graph=False)
            out.setdefault(name, []).append(2.0 * 32 * 32 * 64 * n[0] / ms / 1e9)
    return {k: round(sorted(v)[len(v) // 2], 1) for k, v in out.items()}


def run_llama(workload, device, unquantized=False, sdpa="auto", warmup=3, steps=5):
    """Whole-model step of a Llama configuration with every block linear on the Quartet path: bf16 autocast around
    forward and backward, cross-entropy on random ids, AdamW (fp32 state) for the ~800 M configuration."""
    from quartet_amd import llama as L
    torch.manual_seed(0)
    over = L.unquantized() if unquantized else {}
    over["sdpa_backend"] = sdpa
    if workload == "llama30m":
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

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    torch.cuda.reset_peak_memory_stats()
    t0 = time.perf_counter()
    for _ in range(steps):
        loss = step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / steps * 1e3
    peak_gib = torch.cuda.max_memory_allocated() / 2 ** 30
    lin = sum(m.weight.numel() for _, m in model.block_linears())
    tokens = batch * seq
    out = {"ms_per_step": round(ms, 3), "tokens_per_s": round(tokens / (ms * 1e-3), 1), "final_loss": round(float(loss.detach()), 4),
           "peak_allocated_GiB": round(peak_gib, 2), "block_linear_flops": 6.0 * tokens * lin, "tokens": tokens,
           "what": f"{cfg.n_layer} layers, d {cfg.n_embd}, {batch}x{seq} tokens, {'fwd+bwd+AdamW' if opt_step else 'fwd+bwd'}"}
    del model, opt
    torch.cuda.empty_cache()
    return out


def llama_step(args, device):
    r = run_llama(args.workload, device, args.unquantized, args.sdpa, args.warmup, args.steps)
    flops = r.pop("block_linear_flops")
    ms = r["ms_per_step"]
    return {"metric": "Quartet linear fwd+bwd TFLOPS (MXFP4 MFMA) + Hadamard/quantize HBM GB/s",
            "value": round(flops / (ms * 1e-3) / 1e12, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16" if args.unquantized else "mxfp4", "data": "synthetic",
            "config": {"workload": f"{args.workload}{' (unquantized bf16 linears)' if args.unquantized else ''} whole-model step ({r['what']}); "
                                   f"value counts the block linears' 6*tokens*params flops only ({flops / 1e12:.2f} TFLOP) over the whole step time"},
            "tokens_per_s": r["tokens_per_s"], "final_loss": r["final_loss"], "peak_allocated_GiB": r["peak_allocated_GiB"]}


def llama_blocks(device):
    """The two whole-model configurations in brief: 2 warm-up + 3 timed steps each, the Quartet model and the same model
    with plain bf16 linears beside it."""
    out = {}
    for name in ("llama30m", "llama800m"):
        row = {}
        for label, unq in (("quartet", False), ("bf16_linears", True)):
            r = run_llama(name, device, unquantized=unq, warmup=2, steps=3)
            row["what"] = r["what"]
            row[label] = {"ms_per_step": r["ms_per_step"], "tokens_per_s": r["tokens_per_s"], "peak_allocated_GiB": r["peak_allocated_GiB"]}
        row["speedup_over_bf16_linears"] = round(row["bf16_linears"]["ms_per_step"] / row["quartet"]["ms_per_step"], 3)
        out[name] = row
    return out


def k1536_block(device):
    """The short-K product of the ~800 M model's attention projection (32768 tokens x 4608 out x 1536 in): chain timing
    and the tile-phase stamps, on quest codes of Gaussian operands."""
    from quartet_amd import kernels as K
    M, N, Kd = 32768, 4608, 1536
    g = torch.Generator(device=device).manual_seed(1536)
    x = torch.randn(M, Kd, generator=g, device=device).to(torch.bfloat16)
    w = (0.02 * torch.randn(N, Kd, generator=g, device=device)).to(torch.bfloat16)
    xc, xs, _, _ = K.quantize_mxfp4(x, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=True)
    wc, ws, _, _ = K.quantize_mxfp4(w, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=True)
    ms = sorted(time_kernel(lambda: K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.bfloat16, a_tiled=True, b_tiled=True), reps=20)
                for _ in range(3))[1]
    tf = 2.0 * M * N * Kd / ms / 1e9
    return {"shape": [M, N, Kd], "ms": round(ms, 4), "TFLOPs": round(tf, 1), "frac_of_peak": round(tf / PEAK_FP4_TFLOPS, 4),
            "how": "median of three replays of a 20-launch graph", "tile_phases": gemm_tile_phases(x, w, launches=3)}


def _csrc_sha16():
    """Hash of the kernel sources this build was made from (the traffic profile records the same hash)."""
    import hashlib
    d = os.path.join(ROOT, "quartet_amd", "csrc")
    h = hashlib.sha256()
    for name in sorted(os.listdir(d)):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(d, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()[:16]


def traffic_profile():
    """The tracked byte-counter profile, or None.  `current` says whether the kernel sources are still the ones it
    was measured on."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            prof = json.load(f)
    except (OSError, ValueError):
        return None
    prof["current"] = prof.get("csrc_sha16") == _csrc_sha16()
    return prof


def _traffic_entry(prof, key):
    if prof is None or key not in prof.get("kernels", {}):
        return None, {"file": None}
    k = prof["kernels"][key]
    return float(k["fetch_bytes"] + k["write_bytes"]), {"file": "profiles/hbm_traffic.json", "head": prof.get("head"),
                                                         "matches_this_build": prof["current"],
                                                         "fetch_bytes": k["fetch_bytes"], "write_bytes": k["write_bytes"]}


def counters_to_json(fetch_dir, write_dir, sq_dir=None):
    """Turn the CSV output of the two byte-counter runs

        rocprofv3 --pmc FETCH_SIZE -d <fetch_dir> -o bench --output-format csv -- python3 bench.py --steps 2 --warmup 1 --no-cpu-baseline --no-breakdown --calibration-copy
        rocprofv3 --pmc WRITE_SIZE -d <write_dir> -o bench --output-format csv -- python3 bench.py --steps 2 --warmup 1 --no-cpu-baseline --no-breakdown --calibration-copy

    into profiles/hbm_traffic.json.  The calibration copy (the largest copyBuffer dispatch: 256 MiB read, 256 MiB
    written) fixes how many bytes one counter unit stands for.  With a third directory, the output of

        rocprofv3 --pmc SQ_WAVES SQ_INSTS_VALU ... -d <sq_dir> -o bench --output-format csv -- python3 bench.py --steps 2 --warmup 1 --no-cpu-baseline --no-breakdown --calibration-copy

    adds each kernel's vector instructions per wave (one wave instruction serves 64 lanes; in the quantizers a lane owns
    one group of 32 values per launch, so the figure is also the instructions per group)."""
    import collections
    import csv
    import glob
    import re
    import subprocess

    def read(d, counter=None):
        files = glob.glob(os.path.join(d, "**", "*counter_collection.csv"), recursive=True)
        if not files:
            sys.exit(f"no *counter_collection.csv under {d}")
        agg = collections.defaultdict(list)
        for r in csv.DictReader(open(files[0])):
            if counter is None or r["Counter_Name"] == counter:
                agg[re.sub(r"\(anonymous namespace\)::", "", r["Kernel_Name"])].append(float(r["Counter_Value"]))
        return agg
    fetch, write = read(fetch_dir), read(write_dir)
    valu = read(sq_dir, "SQ_INSTS_VALU") if sq_dir else {}
    waves = read(sq_dir, "SQ_WAVES") if sq_dir else {}
    copy_bytes = 256 << 20

    def unit(agg):
        copies = [v for k, vs in agg.items() if "copyBuffer" in k for v in vs]
        return copy_bytes / max(copies)
    fu, wu = unit(fetch), unit(write)
    groups = {"gemm_mxfp4_tn": lambda k: "gemm_mxfp4_tn" in k and "splitk" not in k and "false, true>" not in k,
              # the instantiation with the masked inverse rotation in its epilogue (the step's two gradient products)
              "gemm_mxfp4_tn_rotated": lambda k: "gemm_mxfp4_tn_big4_kernel" in k and "false, true>" in k,
              "quantize_x_quest_rtn_mask_alone": lambda k: k.startswith("void qm::job_kernel<qm::RowmajorTiledJob") or k.startswith("qm::job_kernel<qm::RowmajorTiledJob"),
              "forward_quantizer_pair": lambda k: "job_pair_kernel<qm::RowmajorTiledJob" in k,
              "gradient_quantizer_pair": lambda k: "job_pair_kernel<qm::TransposedJob" in k,
              "requantizer_pair": lambda k: "job_pair_kernel<qm::RequantJob" in k,
              "inverse_rotation_pair": lambda k: "job_pair_kernel<qm::HadamardBwdJob" in k}
    out = {}
    for name, match in groups.items():
        f = [v for k, vs in fetch.items() if match(k) for v in vs]
        w = [v for k, vs in write.items() if match(k) for v in vs]
        if f and w:
            out[name] = {"fetch_bytes": round(sum(f) / len(f) * fu), "write_bytes": round(sum(w) / len(w) * wu), "dispatches": len(f)}
            vi = [v for k, vs in valu.items() if match(k) for v in vs]
            wv = [v for k, vs in waves.items() if match(k) for v in vs]
            if vi and wv:
                out[name]["valu_instr_per_wave"] = round(sum(vi) / sum(wv), 1)
    head = subprocess.run(["git", "-C", ROOT, "rev-parse", "HEAD"], capture_output=True, text=True).stdout.strip()
    dirty = subprocess.run(["git", "-C", ROOT, "status", "--porcelain", "--", "quartet_amd/csrc"], capture_output=True, text=True).stdout.strip()
    prof = {"what": "HBM-side bytes per launch (mean over the dispatches of a 2-step run) of the isolated linear, tokens 8192 x in 4096 x out 4096",
            "head": head + (" + uncommitted kernel changes" if dirty else ""), "csrc_sha16": _csrc_sha16(),
            "calibration": {"copy_bytes": copy_bytes, "bytes_per_fetch_unit": round(fu, 2), "bytes_per_write_unit": round(wu, 2)},
            "commands": ["rocprofv3 --pmc FETCH_SIZE -d gpurun_out/prof_fetch -o bench --output-format csv -- python3 bench.py --steps 2 --warmup 1 --no-cpu-baseline --no-breakdown --calibration-copy",
                         "rocprofv3 --pmc WRITE_SIZE -d gpurun_out/prof_write -o bench --output-format csv -- python3 bench.py --steps 2 --warmup 1 --no-cpu-baseline --no-breakdown --calibration-copy",
                         "rocprofv3 --pmc SQ_WAVES SQ_WAVE_CYCLES SQ_INSTS_VALU SQ_ACTIVE_INST_VALU SQ_WAIT_INST_ANY SQ_INSTS_VMEM_RD SQ_VALU_MFMA_BUSY_CYCLES SQ_INSTS_MFMA -d gpurun_out/prof_sq -o bench --output-format csv -- python3 bench.py --steps 2 --warmup 1 --no-cpu-baseline --no-breakdown --calibration-copy",
                         "python3 bench.py --counters-to-json gpurun_out/prof_fetch gpurun_out/prof_write gpurun_out/prof_sq"],
            "kernels": out}
    with open(TRAFFIC_PROFILE, "w") as f:
        json.dump(prof, f, indent=1)
        f.write("\n")
    print(json.dumps(prof, indent=1))


def time_layer_steps(step, steps, warmup, sustain_s=1.0):
    """(ms per step over exactly `steps` steps, sustained statistics).  The first figure is the contract's: warm-up, then
    `steps` steps between two synchronisations.  The block is then repeated until `sustain_s` seconds have been spent
    inside timed blocks: the GEMMs run against the chip's power limit, and a window of a few milliseconds after an idle
    period says little about the clock it holds over seconds."""
    for _ in range(warmup):
        step()
    blocks = []
    total = 0.0
    while not blocks or total < sustain_s:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        blocks.append(dt / steps * 1e3)
        total += dt
    srt = sorted(blocks)
    return blocks[0], {"blocks": len(blocks), "steps_per_block": steps, "seconds": round(total, 3),
                       "ms_per_step_median": round(srt[len(srt) // 2], 4), "ms_per_step_min": round(srt[0], 4),
                       "ms_per_step_max": round(srt[-1], 4)}


def make_step(layer, x, dy):
    def step():
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            y = layer(x)
        y.backward(dy)
        x.grad = None
        layer.weight.grad = None
    return step


def gemm_summary(kb, tokens, out_f):
    gemms = [kb[k] for k in ("gemm_fwd", "gemm_dgrad", "gemm_wgrad")]
    ms = sum(g["ms"] for g in gemms) / 3.0
    return ms, 2.0 * tokens * IN_F * out_f / ms / 1e9


def out11008_block(device, args):
    """The configuration's second out-feature count: layer step and the three products (8192x11008x4096,
    8192x4096x11008, 11008x4096x8192), same method as the main figures."""
    out_f = 11008
    x, w, dy = make_inputs(device, out_f=out_f)
    layer = build_layer(device, out_f)
    with torch.no_grad():
        layer.weight.copy_(w)
    x.requires_grad_(True)
    ms, sustained = time_layer_steps(make_step(layer, x, dy), args.steps, args.warmup, sustain_s=0.5)
    flops = 6.0 * T_TOKENS * IN_F * out_f
    x.requires_grad_(False)
    kb = kernel_breakdown(x.detach(), w, dy, only_gemms=True)
    gemm_ms, gemm_tf = gemm_summary(kb, T_TOKENS, out_f)
    return {"workload": f"isolated Quartet linear, tokens {T_TOKENS} x in {IN_F} x out {out_f}", "ms_per_step": round(ms, 4),
            "TFLOPs": round(flops / ms / 1e9, 1), "sustained": sustained, "gemms": kb,
            "gemm_mean": {"ms": round(gemm_ms, 4), "TFLOPs": round(gemm_tf, 1), "frac_of_peak": round(gemm_tf / PEAK_FP4_TFLOPS, 4)}}


def reference_shapes(device):
    """The two layer shapes the reference's notebook reports latencies for (notebooks/benchmark_mxfp4.ipynb: 32768 tokens,
    4096 -> 4096 and 1024 -> 1024, forward and forward + backward, there on another vendor's consumer GPU), timed here
    for this layer and for a plain bf16 linear layer on the same GPU, with the notebook's method in spirit: warm-up, then
    the median of repeated synchronised blocks."""
    import quartet_amd as q
    out = {}
    for tokens, n in ((32768, 4096), (32768, 1024)):
        g = torch.Generator().manual_seed(n)
        x = torch.randn(tokens, n, generator=g).to(torch.bfloat16).to(device).requires_grad_(True)
        dy = (1e-3 * torch.randn(tokens, n, generator=g)).to(torch.bfloat16).to(device)
        layers = {
            "quartet": q.QuantizedLinear(
                n, n, bias=False,
                weight_quantizer=q.QUANTIZER_CLASSES["QuestMXFP4Quantizer"](hadamard_dim=32),
                activation_quantizer=q.QUANTIZER_CLASSES["QuestMXFP4Quantizer"](hadamard_dim=32),
                gradient_quantizer=q.QUANTIZER_CLASSES["AlbertTsengQuantizer"](hadamard_dim=32, stochastic=True, rerotate="signs"),
                backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(device=device, dtype=torch.bfloat16),
            "bf16": torch.nn.Linear(n, n, bias=False).to(device=device, dtype=torch.bfloat16),
        }
        row = {}
        for name, layer in layers.items():
            def fwd():
                with torch.no_grad(), torch.autocast(device_type="cuda", dtype=torch.bfloat16):
                    layer(x)

            def fwd_bwd():
                with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
                    y = layer(x)
                y.backward(dy)
                x.grad = None
                layer.weight.grad = None
            for label, fn in (("fwd_ms", fwd), ("fwd_bwd_ms", fwd_bwd)):
                _, st = time_layer_steps(fn, 10, 3, sustain_s=0.2)
                row[f"{name}_{label}"] = st["ms_per_step_median"]
        row["speedup_fwd"] = round(row["bf16_fwd_ms"] / row["quartet_fwd_ms"], 2)
        row["speedup_fwd_bwd"] = round(row["bf16_fwd_bwd_ms"] / row["quartet_fwd_bwd_ms"], 2)
        row["quartet_fwd_bwd_TFLOPs"] = round(6.0 * tokens * n * n / row["quartet_fwd_bwd_ms"] / 1e9, 1)
        out[f"{tokens}x{n}x{n}"] = row
        del x, dy, layers
    return out


def gemm_shapes(device):
    """The forward and grad-input products of every block linear of the two Llama configurations (32768 tokens), as chains
    of launches on quest codes of Gaussian operands: duration, TFLOP/s, and the rate at which the bf16 output leaves --
    with a short contraction a product is bound by writing its result, not by the matrix pipe."""
    from quartet_amd import kernels as K
    T = 32768
    models = {"llama30m": [(640, 1920), (640, 640), (640, 3456), (1728, 640)],
              "llama800m": [(1536, 4608), (1536, 1536), (1536, 8192), (4096, 1536)]}
    out = {}
    for name, linears in models.items():
        rows = []
        for I, O in linears:
            for what, (M, N, Kd) in (("fwd", (T, O, I)), ("dgrad", (T, I, O))):
                g = torch.Generator(device=device).manual_seed(M + N + Kd)
                tiled = all(d % 128 == 0 and d >= 256 for d in (M, N, Kd))
                a = torch.randn(M, Kd, generator=g, device=device).to(torch.bfloat16)
                b = torch.randn(N, Kd, generator=g, device=device).to(torch.bfloat16)
                ac, as_, _, _ = K.quantize_mxfp4(a, 32, None, K.QM_QUEST_RTN, tiled=tiled)
                bc, bs, _, _ = K.quantize_mxfp4(b, 32, None, K.QM_QUEST_RTN, tiled=tiled)
                del a, b
                ms = sorted(time_kernel(lambda: K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.0, torch.bfloat16, a_tiled=tiled, b_tiled=tiled),
                                        reps=20) for _ in range(3))[1]
                rows.append({"linear": f"{I}->{O}", "product": what, "shape": [M, N, Kd], "ms": round(ms, 4),
                             "TFLOPs": round(2.0 * M * N * Kd / ms / 1e9, 1), "output_GBps": round(M * N * 2 / ms / 1e6, 1)})
        out[name] = rows
    return out


def error_only_scheme_block(device):
    """The two gradient products of scheme "Q(E)W_Q(Et)X" at 8192 x 4096 x 4096: this build's FP4 x bf16 kernel on the
    packed Q(e) / Q(e^T) against the module path the reference takes (de-quantized bf16 Q(e), a transposed copy of e, two
    library bf16 GEMMs), quantizer launches included on both sides."""
    from quartet_amd import kernels as K
    T, I, O = T_TOKENS, IN_F, OUT_F
    g = torch.Generator(device=device).manual_seed(7)
    e = (1e-3 * torch.randn(T, O, generator=g, device=device)).to(torch.bfloat16)
    w = (0.02 * torch.randn(O, I, generator=g, device=device)).to(torch.bfloat16)
    x = torch.randn(T, I, generator=g, device=device).to(torch.bfloat16)
    d = K.FOUR_THIRDS

    def packed():
        ec, es, _, _ = K.quantize_mxfp4(e, 32, None, K.QM_ABSMAX_SR, seed=1)
        K.gemm_mxfp4_bf16_nn(ec, es, w, d)
        etc, ets, _, _ = K.quantize_mxfp4(e, 32, None, K.QM_ABSMAX_SR, transposed_in=True, seed=2)
        K.gemm_mxfp4_bf16_nn(etc, ets, x, d)

    def module_path():
        K.quantize_mxfp4(e, 32, None, K.QM_ABSMAX_SR, seed=1, want_dequant=True)[3] @ w
        K.quantize_mxfp4(e.T.contiguous(), 32, None, K.QM_ABSMAX_SR, seed=2, want_dequant=True)[3] @ x
    ec, es, _, _ = K.quantize_mxfp4(e, 32, None, K.QM_ABSMAX_SR, seed=1)
    etc, ets, _, _ = K.quantize_mxfp4(e, 32, None, K.QM_ABSMAX_SR, transposed_in=True, seed=2)
    fl = 2.0 * T * I * O
    out = {"shape": [T, I, O]}
    for name, fn in (("packed_ms", packed), ("module_path_ms", module_path),
                     ("product_grad_x_ms", lambda: K.gemm_mxfp4_bf16_nn(ec, es, w, d)),
                     ("product_grad_w_ms", lambda: K.gemm_mxfp4_bf16_nn(etc, ets, x, d))):
        out[name] = round(sorted(time_kernel(fn, reps=10) for _ in range(3))[1], 4)
    out["product_grad_x_TFLOPs"] = round(fl / out["product_grad_x_ms"] / 1e9, 1)
    out["product_grad_w_TFLOPs"] = round(fl / out["product_grad_w_ms"] / 1e9, 1)
    out["speedup_over_module_path"] = round(out["module_path_ms"] / out["packed_ms"], 3)
    return out


def quantizer_bounds(prof, x):
    """What else bounds the forward quantizer at this size: its vector-instruction floor (instructions per group from the
    tracked counter profile: a lane owns one group, an instruction occupies its SIMD for four cycles) and what two plain
    library kernels reach on the same tensor with the same timing method (a copy; a sum over four column blocks, which
    reads everything and writes a quarter, about the quantizer's byte mix)."""
    out = {}
    k = (prof or {}).get("kernels", {}).get("quantize_x_quest_rtn_mask_alone", {})
    if "valu_instr_per_wave" in k:
        groups = x.numel() // 32
        lanes = torch.cuda.get_device_properties(x.device).multi_processor_count * 4 * 64
        out["valu_instr_per_group"] = k["valu_instr_per_wave"]
        out["valu_floor_ms_at_2400MHz"] = round(k["valu_instr_per_wave"] * 4 * groups / lanes / 2.4e9 * 1e3, 4)
    rows, cols = x.shape
    dst = torch.empty_like(x)
    quarter = torch.empty(rows, cols // 4, device=x.device, dtype=x.dtype)
    ms_copy = time_kernel_cold(lambda a: (lambda: dst.copy_(a)), [x], reps=8, warmup=1)
    ms_sum = time_kernel_cold(lambda a: (lambda: torch.sum(a.view(rows, 4, cols // 4), dim=1, out=quarter)), [x], reps=8, warmup=1)
    out["library_kernels_same_tensor"] = {"copy_GBps": round(x.numel() * 4 / ms_copy / 1e6, 1),
                                          "sum_of_four_column_blocks_GBps": round(x.numel() * 2.5 / ms_sum / 1e6, 1)}
    return out


def quantizer_sizes_block(device):
    """Quantizer-only configuration in brief: for each tensor size, the slowest and fastest of the nine (mode x Hadamard
    block) cells, HBM-cold."""
    from quartet_amd import kernels as K
    out = {}
    for rows in (4096, 16384, 65536):
        gd = torch.Generator(device=device).manual_seed(rows)
        x = torch.randn(rows, 4096, generator=gd, device=device)
        spike = torch.rand(rows, 4096, generator=gd, device=device) < 1e-3
        x = torch.where(spike, torch.where(torch.rand(rows, 4096, generator=gd, device=device) < 0.5, -1e3, 1e3), x).to(torch.bfloat16)
        cells = []
        for hd in (32, 64, 128):
            for name, mode, mask, bpe in (("quest_rtn_mask", K.QM_QUEST_RTN, True, 2.65625), ("absmax_rtn", K.QM_ABSMAX_RTN, False, 2.53125),
                                          ("absmax_sr", K.QM_ABSMAX_SR, False, 2.53125)):
                ms = time_kernel_cold(lambda a: (lambda: K.quantize_mxfp4(a, hd, None, mode, want_mask=mask, seed=7)), [x], reps=8, warmup=1)
                cells.append((rows * 4096 * bpe / ms / 1e6, f"hd{hd}_{name}"))
        cells.sort()
        out[f"{rows}x4096"] = {"worst": {"cell": cells[0][1], "GBps": round(cells[0][0], 1)},
                               "best": {"cell": cells[-1][1], "GBps": round(cells[-1][0], 1)},
                               "median_GBps": round(cells[len(cells) // 2][0], 1)}
        del x
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=None,
                    help="untimed steps before the timed ones (default 100 for the isolated layer, about 35 ms, and 3 for the model steps: the first steps after an idle period run "
                         "at a clock the chip does not hold; the `sustained` block shows the first timed block beside the median)")
    ap.add_argument("--out-features", type=int, default=OUT_F,
                    help="out features of the isolated layer: 4096 (default, the shape the metric is quoted on) or 11008")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-breakdown", action="store_true")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the blocks the default run appends: out=11008, the K=1536 product, quantizer sizes, the reference's notebook shapes, the two Llama steps")
    ap.add_argument("--workload", default="linear", choices=["linear", "llama30m", "llama800m"],
                    help="linear (default): the isolated 8192x4096x4096 layer the metric is quoted on; llama30m / llama800m: "
                         "whole-model fwd+bwd(+AdamW) step of the 30 M / ~800 M Llama configurations, reported in the same unit "
                         "over the block linears' flops")
    ap.add_argument("--unquantized", action="store_true",
                    help="with a llama workload: identity quantizers and the plain scheme (the bf16 model, for context)")
    ap.add_argument("--sdpa", default="auto", choices=["auto", "default"],
                    help="llama workloads: library attention kernels tried in the model's own order (auto) or the dispatcher's (default)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one plain 256 MiB device copy (a known-traffic kernel for scaling profiler byte counters) and one "
                         "forward quantizer launch on its own")
    ap.add_argument("--counters-to-json", nargs="+", metavar="DIR",
                    help="no GPU work: summarise the CSV output of the two byte-counter runs (FETCH_DIR WRITE_DIR) and, if given, "
                         "of the shader-sequencer counter run (SQ_DIR) into profiles/hbm_traffic.json")
    ap.add_argument("--quantizer-sweep", action="store_true",
                    help="also time the quantizer alone on [rows x 4096] for rows 4096/16384/65536, three modes, hd 32/64/128")
    ap.add_argument("--gemm-operand-content", action="store_true",
                    help="also time the forward GEMM on operands of different content (real codes, random, constant): shows the power limit")
    ap.add_argument("--reference-shapes", action="store_true",
                    help="also time the layer (and a bf16 linear layer, for the ratio) at the two shapes the reference's notebook "
                         "reports: 32768 tokens x 4096 x 4096 and x 1024 x 1024, forward and forward + backward")
    ap.add_argument("--gemm-shapes", action="store_true",
                    help="also time the forward and grad-input products of every block linear of the two Llama configurations")
    ap.add_argument("--library-gemm", action="store_true",
                    help="also time the vendor library's MXFP4 product (torch._scaled_mm) on the forward GEMM's shape, for context")
    args = ap.parse_args()
    if args.counters_to_json:
        if len(args.counters_to_json) not in (2, 3):
            sys.exit("--counters-to-json FETCH_DIR WRITE_DIR [SQ_DIR]")
        counters_to_json(*args.counters_to_json)
        return
    if args.warmup is None:
        args.warmup = 100 if args.workload == "linear" else 3
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the quantized-linear path has no CPU fallback")
    sys.path.insert(0, ROOT)
    device = torch.device("cuda:0")
    if args.workload != "linear":
        print(json.dumps(llama_step(args, device)))
        return
    out_f = args.out_features
    x, w, dy = make_inputs(device, out_f=out_f)
    layer = build_layer(device, out_f)
    with torch.no_grad():
        layer.weight.copy_(w)
    x.requires_grad_(True)
    if args.calibration_copy:
        from quartet_amd import kernels as K
        src = torch.empty(256 << 20, dtype=torch.uint8, device=device).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        K.quantize_mxfp4(x.detach(), 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=True)
        torch.cuda.synchronize()
        del src, dst
    flops = 6.0 * T_TOKENS * IN_F * out_f
    kb = None
    if not args.no_breakdown:
        # The per-kernel timings run first, behind 100 untimed layer steps of their own (about 35 ms): both they and the
        # headline figure below are then taken on a chip that has been busy for a while, as during training, instead of on
        # one that has just left its idle clocks.
        step0 = make_step(layer, x, dy)
        for _ in range(100):
            step0()
        x.requires_grad_(False)
        kb = kernel_breakdown(x.detach(), w, dy)
        x.requires_grad_(True)
    ms_per_step, sustained = time_layer_steps(make_step(layer, x, dy), args.steps, args.warmup,
                                              sustain_s=0.0 if args.calibration_copy else 1.0)
    result = {
        "metric": "Quartet linear fwd+bwd TFLOPS (MXFP4 MFMA) + Hadamard/quantize HBM GB/s",
        "value": round(flops / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "mxfp4", "data": "synthetic",
        "config": {"workload": f"isolated Quartet linear fwd+dgrad+wgrad, tokens {T_TOKENS} x in {IN_F} x out {out_f}, "
                               "bf16 X/W/dY, quest-RTN forward, absmax-SR backward, Hadamard 32"},
        "order": "100 untimed layer steps, per-kernel timings, then warm-up + timed steps (value), then the remaining blocks",
        "sustained": {**sustained, "TFLOPs_median": round(flops / sustained["ms_per_step_median"] / 1e9, 1)},
    }
    prof = traffic_profile() if out_f == OUT_F else None
    if not args.no_breakdown:
        x.requires_grad_(False)
        result["kernels"] = kb
        # The three GEMMs of a step (fwd, dgrad, wgrad) run the same kernel on the same flop count: the roofline entry is
        # their mean duration inside the step, where they run between quantizer kernels (in_step_gemm_ms_by_difference),
        # which is what a profiler's per-kernel average over the step loop shows.  `back_to_back` times each of the three
        # as an unbroken chain of its own launches: that holds the chip at its power limit throughout and is the slowest
        # setting for this kernel (5-10 % longer).
        chain_ms, chain_tf = gemm_summary(kb, T_TOKENS, out_f)
        fused = "epilogue" in kb["gemm_dgrad"]
        diff = in_step_gemm_ms_by_difference(x.detach(), w, dy, fused)
        gemm_ms = diff.pop("ms")
        gemm_tf = 2.0 * T_TOKENS * IN_F * out_f / gemm_ms / 1e9
        traffic, source = _traffic_entry(prof, "gemm_mxfp4_tn")
        if fused and traffic is not None:
            t_rot, _ = _traffic_entry(prof, "gemm_mxfp4_tn_rotated")
            if t_rot is not None:   # per launch, as the step runs them: one plain product, two with the rotation (these also read mask bits)
                source = {**source, "plain_product_bytes": traffic, "rotated_product_bytes": t_rot}
                traffic = round((traffic + 2.0 * t_rot) / 3.0, 1)
        what = "mean of the step's three products, timed inside the step"
        if fused:
            what += ("; the two gradient products carry the masked inverse rotation in their epilogue (flops counted: the product's "
                     "2 M N K only), so the step has no inverse-rotation kernels")
        result["roofline"] = {"bound": "mfma", "kernel": f"gemm_mxfp4_tn ({T_TOKENS}x{out_f}x{IN_F}, {T_TOKENS}x{IN_F}x{out_f}, {out_f}x{IN_F}x{T_TOKENS})",
                              "achieved": round(gemm_tf, 1), "peak": PEAK_FP4_TFLOPS, "unit": "TFLOP/s",
                              "frac": round(gemm_tf / PEAK_FP4_TFLOPS, 4), "traffic": traffic, "traffic_source": source,
                              "avg_launch_ms": round(gemm_ms, 4), "how": {"what": what, **diff},
                              "back_to_back": {"avg_launch_ms": round(chain_ms, 4), "TFLOPs": round(chain_tf, 1),
                                               "frac": round(chain_tf / PEAK_FP4_TFLOPS, 4)}}
        if fused:
            # the same measurement on the composition without the fusion: three plain products and two rotation kernels
            plain = in_step_gemm_ms_by_difference(x.detach(), w, dy, False)
            p_ms = plain.pop("ms")
            p_tf = 2.0 * T_TOKENS * IN_F * out_f / p_ms / 1e9
            result["roofline"]["plain_products"] = {"avg_launch_ms": round(p_ms, 4), "TFLOPs": round(p_tf, 1), "frac": round(p_tf / PEAK_FP4_TFLOPS, 4),
                                                    "how": {"what": "three plain products in a step that rotates with kernels of its own", **plain}}
        qk = kb["quantize_x_quest_rtn_mask"]
        traffic, source = _traffic_entry(prof, "quantize_x_quest_rtn_mask_alone")
        result["roofline_quantize"] = {"bound": "hbm", "kernel": f"quantize_rowmajor (quest RTN + mask, {T_TOKENS}x{IN_F} bf16)",
                                       "achieved": qk["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                       "frac": round(qk["GBps"] / PEAK_HBM_GBS, 4), "traffic": traffic, "traffic_source": source,
                                       "avg_launch_ms": qk["ms"], **quantizer_bounds(prof, x.detach())}
    if not args.no_breakdown:
        result["roofline"]["tile_phases"] = gemm_tile_phases(x.detach(), w)
        ceil = mfma_only_ceiling(x.detach(), w)
        result["mfma_only_TFLOPs"] = ceil
        result["roofline"]["frac_of_mfma_only_rate_on_real_operands"] = round(
            result["roofline"]["achieved"] / ceil["quest_rtn_codes_of_the_forward_operands"], 4)
    if not args.no_extra and not args.no_breakdown and out_f == OUT_F:
        del layer
        result["out11008"] = out11008_block(device, args)
        result["k1536"] = k1536_block(device)
        result["quantizer_sizes"] = quantizer_sizes_block(device)
        result["reference_shapes"] = reference_shapes(device)
        result["error_only_scheme"] = error_only_scheme_block(device)
        del x, w, dy
        torch.cuda.empty_cache()
        result["llama"] = llama_blocks(device)
        x, w, dy = make_inputs(device, out_f=out_f)
    if args.quantizer_sweep:
        result["quantizer_sweep"] = quantizer_sweep(device)
    if args.reference_shapes and "reference_shapes" not in result:
        result["reference_shapes"] = reference_shapes(device)
    if args.gemm_shapes:
        result["gemm_shapes"] = gemm_shapes(device)
    if args.library_gemm:
        result["library_gemm"] = library_gemm(device)
    if args.gemm_operand_content:
        result["gemm_operand_content"] = gemm_operand_content(x.detach(), w, dy)
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(out_f=out_f)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
