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


def time_kernel(fn, reps=20, warmup=3):
    """Average duration (ms) of one launch sequence `fn`, HIP events on the stream the kernels run on."""
    for _ in range(warmup):
        fn()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(reps):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / reps


def kernel_breakdown(x, w, dy):
    """Per-kernel timings of the twelve launches of one step, with algorithmic bytes / flops."""
    from quartet_amd import kernels as K
    T, I, O = x.shape[0], x.shape[1], w.shape[0]
    out = {}
    xc, xs, xm, _ = K.quantize_mxfp4(x, 32, None, K.QM_QUEST_RTN, want_mask=True)
    wc, ws, wm, _ = K.quantize_mxfp4(w, 32, None, K.QM_QUEST_RTN, want_mask=True)
    signs = 0x5A5AA5A5
    ec, es, _, _ = K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, seed=1)
    etc, ets, _, _ = K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, transposed_in=True, seed=2)
    wtc, wts, _ = K.requantize_transposed_mxfp4(wc, ws, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=3)
    xtc, xts, _ = K.requantize_transposed_mxfp4(xc, xs, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=4)
    gxq = K.gemm_mxfp4_tn(ec, es, wtc, wts, 1.0, torch.bfloat16)
    gwq = K.gemm_mxfp4_tn(etc, ets, xtc, xts, 1.0, torch.bfloat16)

    def hbm(name, elems, bytes_per_elem, fn):
        ms = time_kernel(fn)
        out[name] = {"ms": round(ms, 4), "GBps": round(elems * bytes_per_elem / ms / 1e6, 1),
                     "bytes_per_elem": bytes_per_elem}

    def mfma(name, m, n, k, fn):
        ms = time_kernel(fn)
        out[name] = {"ms": round(ms, 4), "TFLOPs": round(2.0 * m * n * k / ms / 1e9, 1), "shape": [m, n, k]}

    hbm("quantize_x_quest_rtn_mask", T * I, 2.65625, lambda: K.quantize_mxfp4(x, 32, None, K.QM_QUEST_RTN, want_mask=True))
    hbm("quantize_w_quest_rtn_mask", O * I, 2.65625, lambda: K.quantize_mxfp4(w, 32, None, K.QM_QUEST_RTN, want_mask=True))
    mfma("gemm_fwd", T, O, I, lambda: K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.bfloat16))
    hbm("quantize_e_absmax_sr", T * O, 2.53125, lambda: K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, seed=1))
    hbm("quantize_et_absmax_sr_transposed", T * O, 2.53125,
        lambda: K.quantize_mxfp4(dy, 32, signs, K.QM_ABSMAX_SR, transposed_in=True, seed=2))
    hbm("requantize_wt", O * I, 1.0625,
        lambda: K.requantize_transposed_mxfp4(wc, ws, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=3))
    hbm("requantize_xt", T * I, 1.0625,
        lambda: K.requantize_transposed_mxfp4(xc, xs, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=4))
    mfma("gemm_dgrad", T, I, O, lambda: K.gemm_mxfp4_tn(ec, es, wtc, wts, 1.0, torch.bfloat16))
    mfma("gemm_wgrad", O, I, T, lambda: K.gemm_mxfp4_tn(etc, ets, xtc, xts, 1.0, torch.bfloat16))
    hbm("hadamard_bwd_x", T * I, 4.125, lambda: K.masked_hadamard_bwd(gxq, 32, torch.bfloat16, None, xm))
    hbm("hadamard_bwd_w", O * I, 4.125, lambda: K.masked_hadamard_bwd(gwq, 32, torch.bfloat16, None, wm))
    return out


def cpu_baseline(sample_tokens=2048):
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
    dt = time.perf_counter() - t0
    assert y.shape[0] == sample_tokens and gx.shape == (sample_tokens, IN_F) and gw.shape == (OUT_F, IN_F)
    flops = 6.0 * sample_tokens * IN_F * OUT_F
    return {"value": round(flops / dt / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"one fwd+bwd on the first {sample_tokens} of {T_TOKENS} tokens (same I={IN_F}, O={OUT_F}); "
                      f"CPU oracle quantizers + fp32 BLAS matmuls on de-quantized operands, {dt:.2f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-breakdown", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X: this build has no multi-GPU path (run with --gpus 1)")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the quantized-linear path has no CPU fallback")
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
    device = torch.device("cuda:0")
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
        g = kb["gemm_fwd"]
        gemm_ms = g["ms"]
        result["roofline"] = {"bound": "mfma", "kernel": "gemm_mxfp4_tn (fwd 8192x4096x4096)",
                              "achieved": g["TFLOPs"], "peak": PEAK_FP4_TFLOPS, "unit": "TFLOP/s",
                              "frac": round(g["TFLOPs"] / PEAK_FP4_TFLOPS, 4), "traffic": None,
                              "avg_launch_ms": gemm_ms}
        qk = kb["quantize_x_quest_rtn_mask"]
        result["roofline_quantize"] = {"bound": "hbm", "kernel": "quantize_rowmajor (quest RTN + mask, 8192x4096 bf16)",
                                       "achieved": qk["GBps"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                       "frac": round(qk["GBps"] / PEAK_HBM_GBS, 4), "traffic": None,
                                       "avg_launch_ms": qk["ms"]}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
