"""Pins of the oracle's producer functions (RMSNorm and the SwiGLU product in front of the activation quantizer,
src/models/llama.py:64-75,113-114 of the reference) against float64 evaluations of the reference's formulas, the C
library and closed forms -- none of them shares code with the oracle."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as o


def ulp32(t):
    return float(np.spacing(np.float32(abs(t))))


def test_exp_against_the_c_library():
    rng = np.random.default_rng(0)
    zs = np.concatenate([rng.uniform(-87.0, 88.7, 20000), rng.normal(0.0, 2.0, 20000), [0.0, -0.0, 1.0, -1.0, 88.0, -87.0]])
    worst = 0.0
    for z in zs.astype(np.float32):
        t = math.exp(float(z))
        worst = max(worst, abs(float(o.exp_fixed(z)) - t) / ulp32(t))
    assert worst <= 1.5, worst
    assert o.exp_fixed(0.0) == 1.0 and o.exp_fixed(100.0) == np.inf and o.exp_fixed(-200.0) == 0.0
    assert np.isnan(o.exp_fixed(np.nan))


def test_silu_against_float64_and_limits():
    rng = np.random.default_rng(1)
    for x in np.concatenate([rng.normal(0.0, 4.0, 20000), rng.uniform(-100, 100, 2000)]).astype(np.float32):
        t = float(x) / (1.0 + math.exp(-float(x)))
        if x < -88.0:   # e^-x overflows fp32 there, as it does in torch: the quotient is -0 instead of ~1e-37
            assert abs(float(o.silu(x))) <= abs(t) * (1 + 1e-6)
            continue
        assert abs(float(o.silu(x)) - t) <= 2.5 * ulp32(t), (x, o.silu(x), t)
    assert o.silu(0.0) == 0.0
    assert o.silu(200.0) == 200.0                                  # 1 + e^-200 rounds to 1
    got = o.silu(-200.0)
    assert got == 0.0 and np.signbit(got)                          # x / inf
    assert o.silu(1.0) == np.float32(1.0 / (1.0 + math.exp(-1.0)))


def test_silu_on_every_bf16_input_against_torch():
    """Rounded to bf16, the fixed-sequence silu agrees with torch's own bf16 silu on (nearly) every input: the two
    differ only where their fp32 values, one ulp apart, straddle a bf16 rounding boundary."""
    bits = np.arange(65536, dtype=np.uint16)
    x = o.bf16_bits_to_f32(bits)
    keep = np.isfinite(x)
    h12 = np.stack([bits[keep], np.full(keep.sum(), 0x3F80, dtype=np.uint16)], axis=0).reshape(1, -1)  # gate = 1.0
    mine = o.swiglu(np.ascontiguousarray(h12))[0]
    theirs = F.silu(torch.from_numpy(x[keep]).to(torch.bfloat16)).view(torch.int16).numpy().view(np.uint16)
    nz = (mine & 0x7FFF) != 0                                       # signs of zero results aside
    assert np.count_nonzero(mine[nz] != theirs[nz]) <= 8
    a = o.bf16_bits_to_f32(mine[nz]).astype(np.float64)
    b = o.bf16_bits_to_f32(theirs[nz]).astype(np.float64)
    assert np.all(np.abs(a - b) <= 2.0 ** -7 * np.abs(b))            # never more than one bf16 step


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
@pytest.mark.parametrize("rows,cols", [(7, 32), (5, 640), (3, 1536), (2, 4096)])
def test_rmsnorm_against_float64(dtype, rows, cols):
    rng = np.random.default_rng(rows * cols)
    x = (rng.standard_normal((rows, cols)) * rng.uniform(0.1, 30.0, (rows, 1))).astype(np.float32)
    gain = rng.uniform(0.5, 1.5, cols).astype(np.float32)
    xin = o.f32_to_bf16_bits(x) if dtype == "bf16" else x
    xv = o.bf16_bits_to_f32(xin).astype(np.float64) if dtype == "bf16" else x.astype(np.float64)
    eps = 1e-5
    out, factor = o.rmsnorm(xin, gain, eps)
    want_f = 1.0 / np.sqrt((xv ** 2).mean(axis=1) + eps)
    assert np.all(np.abs(factor - want_f) <= 2e-7 * want_f)
    normed = xv * want_f[:, None]
    if dtype == "bf16":   # .type_as(x): one bf16 rounding before the gain
        tol = 2.0 ** -8
    else:
        tol = 4e-7
    want = normed * gain.astype(np.float64)
    assert np.all(np.abs(out - want) <= tol * np.abs(want) + 1e-30)
    # the reference's own line, evaluated by torch in the tensor's dtype
    tx = torch.from_numpy(xv.astype(np.float32))
    tx = tx.to(torch.bfloat16) if dtype == "bf16" else tx
    ref = (tx.float() * torch.rsqrt(tx.float().pow(2).mean(-1, keepdim=True) + eps)).type_as(tx) * torch.from_numpy(gain)
    assert ref.dtype == torch.float32
    mismatch = np.abs(out - ref.numpy()) > tol * np.abs(ref.numpy()) + 1e-30
    assert not mismatch.any()


def test_rmsnorm_closed_forms():
    cols, eps = 96, 1e-5
    gain = np.ones(cols, dtype=np.float32)
    x = np.zeros((3, cols), dtype=np.float32)
    x[1] = 3.0                                                     # constant row: mean(x^2) = 9 exactly
    x[2, 5] = -8.0                                                 # one-hot row: mean = 64 / 96
    out, factor = o.rmsnorm(x, gain, eps)
    assert factor[0] == np.float32(1.0) / np.sqrt(np.float32(eps))
    assert factor[1] == np.float32(1.0) / np.sqrt(np.float32(9.0) + np.float32(eps))
    assert factor[2] == np.float32(1.0) / np.sqrt(np.float32(64.0) / np.float32(96.0) + np.float32(eps))
    assert np.all(out[0] == 0.0) and np.all(out[1] == np.float32(3.0) * factor[1])
    assert out[2, 5] == np.float32(-8.0) * factor[2] and np.count_nonzero(out[2]) == 1
    # a permutation of whole 32-element groups among the sixteen partial sums may change rounding, never the value much;
    # scaling the row by a power of two scales the sum of squares exactly (eps = 0)
    rng = np.random.default_rng(3)
    y = rng.standard_normal((1, 1536)).astype(np.float32)
    _, f1 = o.rmsnorm(y, np.ones(1536, dtype=np.float32), 0.0)
    _, f2 = o.rmsnorm(4.0 * y, np.ones(1536, dtype=np.float32), 0.0)
    assert f2[0] == f1[0] / np.float32(4.0)


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_swiglu_against_torch(dtype):
    rng = np.random.default_rng(5)
    rows, hidden = 6, 160
    h = (rng.standard_normal((rows, 2 * hidden)) * 3.0).astype(np.float32)
    hin = o.f32_to_bf16_bits(h) if dtype == "bf16" else h
    got = o.swiglu(hin)
    t = torch.from_numpy(o.bf16_bits_to_f32(hin) if dtype == "bf16" else h)
    t = t.to(torch.bfloat16) if dtype == "bf16" else t
    up, gate = t.split(hidden, dim=-1)                              # up first, then gate (llama.py:113)
    want = (F.silu(up) * gate).float().numpy()
    gotf = o.bf16_bits_to_f32(got) if dtype == "bf16" else got
    tol = 2.0 ** -7 if dtype == "bf16" else 1e-6
    assert np.all(np.abs(gotf - want) <= tol * np.abs(want) + 1e-30)
    if dtype == "bf16":
        assert np.mean(gotf != want) < 0.01                         # bit-identical almost everywhere
    # swapping the halves must change the result (the order of up and gate is part of the contract)
    swapped = np.concatenate([hin[:, hidden:], hin[:, :hidden]], axis=1)
    assert not np.array_equal(o.swiglu(np.ascontiguousarray(swapped)), got)
