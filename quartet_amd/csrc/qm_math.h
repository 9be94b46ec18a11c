// Scalar arithmetic shared by the HIP kernels: everything here is plain IEEE fp32 / integer code
// that also compiles as host C++ (g++), so the rounding rules can be checked exhaustively on a
// CPU against the test oracle.  Arithmetic follows the reference kernel
// src/models/quantization/quantizers/mxfp4_triton.py:51-165 (scale rules, strict-threshold RTN,
// bracketed stochastic rounding, sign = "not (t > 0)", clip mask |t| < 6).
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define QM_HD __host__ __device__ __forceinline__
#else
#define QM_HD inline
#endif

namespace qm {

enum Mode : int { QUEST_RTN = 0, ABSMAX_RTN = 1, ABSMAX_SR = 2, QUEST_SR = 3 };
enum DType : int { BF16 = 0, F32 = 1 };

QM_HD uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
QM_HD float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

QM_HD float bf16_to_f32(uint16_t h) { return u2f((uint32_t)h << 16); }
// round-to-nearest-even; NaN stays a quiet NaN
QM_HD uint16_t f32_to_bf16(float f) {
    uint32_t b = f2u(f);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x40);
    b += 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}

// fl32(2.92247856 / 6.0)  (mxfp4.py:137) and fl32(1 / 0.75) (mxfp4_triton.py:60)
constexpr float kQuestG = (float)(2.92247856 / 6.0);
constexpr float kFourThirds = (float)(1.0 / 0.75);

// hd^-1/2 rounded to the tensor's dtype (mxfp4.py:42-44,49)
QM_HD float hadamard_scale(int hd, int dtype) {
    float c = hd == 32 ? 0.17677669529663687f : (hd == 64 ? 0.125f : 0.08838834764831845f);
    if (dtype == BF16) c = bf16_to_f32(f32_to_bf16(c));
    return c;
}

// exact 2^e as fp32 for e in [-149, 127]
QM_HD float pow2i(int e) {
    return e >= -126 ? u2f((uint32_t)(e + 127) << 23) : u2f(1u << (e + 149));
}

// x * 2^e, correctly rounded; two exact-or-single-rounding multiplies, valid for |e| <= 252 as
// long as the first factor does not round (it is applied to the smaller half of the shift).
QM_HD float scale_pow2(float x, int e) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_ldexpf(x, e);
#else
    return __builtin_ldexpf(x, e);
#endif
}

// IEEE round-to-nearest g / fl32(4/3) without a hardware divide: fl32(3/4) is the correctly
// rounded reciprocal of 0x3FAAAAAB, so one residual correction gives the correctly rounded
// quotient for |g| >= 2^-104 (checked over every fp32 bit pattern on the host; below that the
// residual loses bits to underflow, the result keeps g's sign and stays non-zero).
QM_HD float div_four_thirds(float g) {
    float q0 = g * 0.75f;
    float r = __builtin_fmaf(-q0, kFourThirds, g);
    return __builtin_fmaf(r, 0.75f, q0);
}

// The same quotient in two operations for |g| >= 2^-100 (and for zeros up to the sign of zero): fl32(4/3) is exactly
// (4/3)(1 + 2^-25), so 1/fl32(4/3) = 3/4 - 3/2 * 2^-26 + O(2^-50) and one fma over the rounded low part is correctly
// rounded (checked over every fp32 bit pattern on the host; below 2^-100 the low part loses bits to underflow, the
// result keeps g's sign and stays non-zero).
constexpr float kInvFourThirdsLo = -0x1.8p-26f;
QM_HD float div_four_thirds_fast(float g) { return __builtin_fmaf(g, 0.75f, g * kInvFourThirdsLo); }

// RTN onto the E2M1 magnitudes {0,.5,1,1.5,2,3,4,6}: strict '>' against the seven midpoints,
// i.e. ties go toward zero and anything above 5 saturates at 6 (mxfp4_triton.py:131-159).
QM_HD int rtn_code(float A) {
    int c = 0;
    c += A > 0.25f;
    c += A > 0.75f;
    c += A > 1.25f;
    c += A > 1.75f;
    c += A > 2.5f;
    c += A > 3.5f;
    c += A > 5.0f;
    return c;
}

QM_HD float e2m1_value(int mag) {
    // 0, .5, 1, 1.5, 2, 3, 4, 6
    return mag < 2 ? 0.5f * (float)mag : u2f(((uint32_t)((mag >> 1) + 126) << 23) | ((uint32_t)(mag & 1) << 22));
}

// SR (mxfp4_triton.py:70-129): bracket by strict '>' against {.5,1,1.5,2,3,4}, p = (A-lo)/(hi-lo),
// up iff u < p.  hi-lo is a power of two and A-lo is exact, so p is exact.
QM_HD int sr_code(float A, float u) {
    int lo = 0;
    lo += A > 0.5f;
    lo += A > 1.0f;
    lo += A > 1.5f;
    lo += A > 2.0f;
    lo += A > 3.0f;
    lo += A > 4.0f;
    float vlo = e2m1_value(lo), vhi = e2m1_value(lo + 1);
    float p = (A - vlo) / (vhi - vlo);
    return lo + (u < p ? 1 : 0);
}

// ---- SiLU with a fixed instruction sequence ------------------------------------------------------------------
// e^z from n = rint(z log2 e), r = z - n ln2 (two-constant reduction, fused), the degree-7 Taylor polynomial in r
// (|r| <= 0.347: truncation error below 2^-27) and an exact scaling by 2^n: the same fmas on the CPU and on the GPU,
// about one ulp from the exact value.  Above ln(FLT_MAX) the result is +inf; NaN passes through.
QM_HD float exp_fixed(float z) {
    if (!(z == z)) return z;
    if (z > 88.72283935546875f) return u2f(0x7f800000u);
    if (z < -104.0f) return 0.0f;
    const float n = __builtin_rintf(z * 1.44269502162933349609375f);
    float r = __builtin_fmaf(n, -0.693145751953125f, z);
    r = __builtin_fmaf(n, -1.428606765330187045037746429443359375e-06f, r);
    float p = 1.0f / 5040.0f;
    p = __builtin_fmaf(p, r, 1.0f / 720.0f);
    p = __builtin_fmaf(p, r, 1.0f / 120.0f);
    p = __builtin_fmaf(p, r, 1.0f / 24.0f);
    p = __builtin_fmaf(p, r, 1.0f / 6.0f);
    p = __builtin_fmaf(p, r, 0.5f);
    p = __builtin_fmaf(p, r, 1.0f);
    p = __builtin_fmaf(p, r, 1.0f);
    return scale_pow2(p, (int)n);
}
// x / (1 + e^-x), the form torch.nn.functional.silu evaluates (src/models/llama.py:113 of the reference calls it)
QM_HD float silu_fixed(float x) { return x / (1.0f + exp_fixed(-x)); }

// ---- Philox4x32-7 (Random123; the fewest rounds it publishes as passing its test batteries) ------------------
struct Philox4 {
    uint32_t w[4];
};
template <int ROUNDS>
QM_HD Philox4 philox4x32(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
        // one 32x32->64 multiply each (v_mad_u64_u32 on the GPU)
        const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        c0 = n0; c1 = (uint32_t)p1; c2 = n2; c3 = (uint32_t)p0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    Philox4 o;
    o.w[0] = c0; o.w[1] = c1; o.w[2] = c2; o.w[3] = c3;
    return o;
}
constexpr int kPhiloxRounds = 7;
// Random bits of element `o` (flat offset in the tensor being quantized): one Philox call per sixteen consecutive
// elements, counter = o/16.  Element j of the sixteen reads word j/4 rotated left by 8 * (j%4) bits and takes its top 22
// bits as the field f: each element of a word has its own most significant byte and shares the bytes below with the
// word's other elements at lower significance.  Its uniform is the largest float below (2^22 - f) * 2^-22: "u < p" is
// then exactly "floor(p * 2^22) + f carries out of 22 bits", which is what the hardware's stochastic-rounding convert
// evaluates with f as its random field.
QM_HD uint32_t rotl32(uint32_t w, int s) { return s ? ((w << s) | (w >> (32 - s))) : w; }
QM_HD uint32_t philox_field22(const Philox4& p, int j) { return rotl32(p.w[j >> 2], 8 * (j & 3)) >> 10; }
QM_HD float uniform_from_field22(uint32_t f) {
    return u2f(f2u((float)(4194304u - f) * (1.0f / 4194304.0f)) - 1u);
}
QM_HD Philox4 philox_for_hexadecad(uint64_t seed, uint64_t block16) {
    return philox4x32<kPhiloxRounds>((uint32_t)block16, (uint32_t)(block16 >> 32), 0u, 0u, (uint32_t)seed, (uint32_t)(seed >> 32));
}

}  // namespace qm
