"""Writes tests/golden/exact_vectors.json: golden vectors for the rotate + MXFP4-quantize path.

The reference (IST-DASLab/Quartet) holds no test vectors for this path, so these are worked out from its formulas
(src/models/quantization/quantizers/mxfp4_triton.py:44-165) with exact rational arithmetic -- `fractions.Fraction`
everywhere a decision is taken -- by a script that shares no code with `oracle/` or with the kernels.  Inputs are
chosen so that nothing depends on a summation order or on an approximate transcendental:

  * x = S y with small integers y (S = Sylvester matrix): every partial sum of the rotation is an integer, and
    c * hd (c = hd^-1/2 rounded to the tensor's dtype) is a short dyadic rational for bf16 tensors and for hd = 64,
    so the rotated values are exact whatever order a kernel adds in;
  * quest scale: the exponent floor(log2(G * std + 1e-8)) is taken from a high-precision evaluation and the case is
    rejected unless the argument sits at least 1e-3 (relative) away from a power of two;
  * absmax scale: floor(log2 max|v|) - 2 is exact; t = v / (2^k * fl32(4/3)) is rounded to fp32 exactly;
  * rounding: strict comparisons against the seven midpoints (ties toward zero), or the bracketed stochastic rule with
    explicit uniforms u that are multiples of 2^-10, p = (A - lo) / (hi - lo) compared exactly;
  * sign bit = "not (t > 0)", clip mask = |t| < 6.

Run from the repository root:  python tests/golden/make_exact_vectors.py
"""
import json
import os
import random
import struct
from decimal import Decimal, getcontext
from fractions import Fraction

QUEST_RTN, ABSMAX_RTN, ABSMAX_SR, QUEST_SR = 0, 1, 2, 3
GRID = [Fraction(0), Fraction(1, 2), Fraction(1), Fraction(3, 2), Fraction(2), Fraction(3), Fraction(4), Fraction(6)]
MIDPOINTS = [Fraction(1, 4), Fraction(3, 4), Fraction(5, 4), Fraction(7, 4), Fraction(5, 2), Fraction(7, 2), Fraction(5)]
FOUR_THIRDS = Fraction(struct.unpack("<f", struct.pack("<I", 0x3FAAAAAB))[0])   # fl32(1 / 0.75)
QUEST_G = Fraction(struct.unpack("<f", struct.pack("<I", 0x3EF96285))[0])      # fl32(2.92247856 / 6.0)
EPS = Fraction(struct.unpack("<f", struct.pack("<f", 1e-8))[0])                # fl32(1e-8)
getcontext().prec = 60


def floor_log2(q):
    e = q.numerator.bit_length() - q.denominator.bit_length()
    while Fraction(2) ** e > q:
        e -= 1
    while Fraction(2) ** (e + 1) <= q:
        e += 1
    return e


def round_to_f32(q):
    """Nearest fp32 (ties to even) of a rational in the normal range."""
    if q == 0:
        return Fraction(0)
    a = abs(q)
    e = floor_log2(a)
    assert -126 <= e <= 127
    ulp = Fraction(2) ** (e - 23)
    n = a / ulp
    fl = n.numerator // n.denominator
    rem = n - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return (fl * ulp) * (1 if q > 0 else -1)


def hadamard_constant(hd, dtype):
    """hd^-1/2 in the tensor's dtype (quantizers/mxfp4.py:42-49): bf16(32^-1/2) = 181/1024, bf16(128^-1/2) = 181/2048,
    64^-1/2 = 1/8 in either dtype.  fp32 tensors are only used with hd = 64 here (see the module docstring)."""
    if hd == 64:
        return Fraction(1, 8)
    assert dtype == "bf16"
    return {32: Fraction(181, 1024), 128: Fraction(181, 2048)}[hd]


def fits_bf16(n):
    """Is the integer n a bf16 value (at most 8 significant bits)?"""
    n = abs(n)
    while n and n % 2 == 0:
        n //= 2
    return n < 256


def sylvester_entry(i, j):
    return -1 if bin(i & j).count("1") & 1 else 1


def rtn_mag(A):
    return sum(1 for m in MIDPOINTS if A > m)


def sr_mag(A, u):
    lo = sum(1 for b in GRID[1:7] if A > b)          # strict '>' against .5 1 1.5 2 3 4
    p = (A - GRID[lo]) / (GRID[lo + 1] - GRID[lo])
    return lo + (1 if u < p else 0)


def quantize_group(v, mode, u):
    """v: 32 exact rotated values -> (e8m0 byte, [nibble], [mask bit])."""
    quest = mode in (QUEST_RTN, QUEST_SR)
    if quest:
        m = sum(v) / 32
        var = sum(x * x for x in v) / 32 - m * m
        std = Decimal(var.numerator) / Decimal(var.denominator)
        s = Decimal(QUEST_G.numerator) / Decimal(QUEST_G.denominator) * std.sqrt() + Decimal(EPS.numerator) / Decimal(EPS.denominator)
        E = int((s.ln() / Decimal(2).ln()).to_integral_value(rounding="ROUND_FLOOR"))
        lo, hi = Decimal(2) ** E, Decimal(2) ** (E + 1)
        if not (lo * Decimal("1.001") < s < hi * Decimal("0.999")):
            return None                               # too close to an exponent boundary: not a fixture
        t = [x / Fraction(2) ** E for x in v]
        byte = E + 127
    else:
        a = max(abs(x) for x in v)
        if a == 0:
            # the reference produces NaN -> every comparison false -> -0.0; this build's documented choice of the
            # (irrelevant) scale byte for such a group is 0
            return 0, [8] * 32, [1] * 32
        k = floor_log2(a) - 2
        t = [round_to_f32((x / Fraction(2) ** k) / FOUR_THIRDS) for x in v]
        byte = k + 127
    assert 0 < byte < 255
    nibbles, keep = [], []
    for i, ti in enumerate(t):
        A = abs(ti)
        mag = sr_mag(A, u[i]) if mode in (ABSMAX_SR, QUEST_SR) else rtn_mag(A)
        nibbles.append(min(mag, 7) | (0 if ti > 0 else 8))
        keep.append(1 if A < 6 else 0)
    return byte, nibbles, keep


def f32_bits(q):
    return struct.unpack("<I", struct.pack("<f", float(q)))[0]


def make_case(rng, name, hd, dtype, mode, with_signs, rows=2, chunks=2, spread=3, outliers=False):
    cols = hd * chunks
    for _ in range(200):
        signs = [rng.choice((-1, 1)) for _ in range(hd)] if with_signs else None
        c = hadamard_constant(hd, dtype)
        xs, us, codes, scales, mask = [], [], [], [], []
        ok = True
        for r in range(rows):
            for ch in range(chunks):
                zero_chunk = (r == 0 and ch == 1 and mode in (ABSMAX_RTN, ABSMAX_SR))
                # y: the rotated vector in units of c * hd; sparse large entries make clipped and saturated values
                y = [0] * hd if zero_chunk else [rng.choice((0, 0, 1, -1, 1, -1, 2, -2, spread, -spread)) for _ in range(hd)]
                if not zero_chunk and outliers:
                    y[rng.randrange(hd)] = rng.choice((-8, 8))
                x = [sum(sylvester_entry(k, j) * y[j] for j in range(hd)) for k in range(hd)]
                if dtype == "bf16" and not all(fits_bf16(v) for v in x):
                    ok = False
                v = [(signs[j] if signs else 1) * c * hd * y[j] for j in range(hd)]
                assert all(round_to_f32(t) == t for t in v), "c * hd * y must be exact in fp32"
                u = [Fraction(rng.randrange(0, 1024), 1024) for _ in range(hd)]
                for g in range(hd // 32):
                    out = quantize_group(v[32 * g:32 * g + 32], mode, u[32 * g:32 * g + 32])
                    if out is None:
                        ok = False
                        break
                    scales.append(out[0]); codes += out[1]; mask += out[2]
                xs += x; us += u
        if ok:
            x_bits = [f32_bits(Fraction(v)) >> (16 if dtype == "bf16" else 0) for v in xs]
            return dict(name=name, hd=hd, dtype=dtype, mode=mode, rows=rows, cols=cols, signs=signs, x_bits=x_bits,
                        u_bits=[f32_bits(v) for v in us] if mode in (ABSMAX_SR, QUEST_SR) else None,
                        nibbles=codes, scales=scales, mask=mask if mode == QUEST_RTN else None)
    raise RuntimeError(f"no admissible inputs found for {name}")


def main():
    rng = random.Random(20240607)
    cases = []
    for dtype, hds in (("bf16", (32, 64, 128)), ("f32", (64,))):
        for hd in hds:
            spread = 3 if hd < 128 else 2
            for mode, mname in ((QUEST_RTN, "quest_rtn"), (ABSMAX_RTN, "absmax_rtn"), (ABSMAX_SR, "absmax_sr"), (QUEST_SR, "quest_sr")):
                for with_signs in (False, True):
                    name = f"{dtype}_hd{hd}_{mname}{'_signs' if with_signs else ''}"
                    cases.append(make_case(rng, name, hd, dtype, mode, with_signs, spread=spread, outliers=with_signs))
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "exact_vectors.json")
    with open(path, "w") as f:
        json.dump(dict(format="x_bits: bf16 or fp32 bit patterns, row-major [rows, cols]; nibbles: E2M1 code per element (bit 3 = sign); "
                              "scales: E8M0 byte per 32 elements; mask: clip-mask bit per element (quest_rtn only); u_bits: fp32 uniforms",
                       cases=cases), f, separators=(",", ":"))
    print(f"wrote {len(cases)} cases to {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
