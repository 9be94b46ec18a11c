// Host build of the kernels' scalar arithmetic (quartet_amd/csrc/qm_math.h) checked against IEEE-754 arithmetic of the
// host compiler.  Built and run by tests/test_host_math.py; prints one line per failed property and exits non-zero.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>

#include "qm_math.h"

using namespace qm;

static int failures = 0;
static void fail(const char* what, uint32_t bits) {
    if (failures++ < 20) std::printf("FAIL %s at 0x%08x\n", what, bits);
}

static void check_division(uint32_t b) {
    const float g = u2f(b);
    if (std::isnan(g) || std::isinf(g)) return;
    volatile float d = kFourThirds;
    const float want = g / d;  // correctly rounded by the host
    const uint32_t mag = b & 0x7fffffffu;
    if (mag >= (23u << 23)) {  // |g| >= 2^-104
        if (f2u(div_four_thirds(g)) != f2u(want)) fail("div_four_thirds", b);
    } else if (mag != 0) {
        const float got = div_four_thirds(g);
        if (got == 0.0f || std::signbit(got) != std::signbit(g)) fail("div_four_thirds sign", b);
    }
    if (mag >= (27u << 23)) {  // |g| >= 2^-100
        if (f2u(div_four_thirds_fast(g)) != f2u(want)) fail("div_four_thirds_fast", b);
    } else if (mag != 0) {
        // below the exact range the fast form may be off in the last bits but never changes sign or becomes zero
        const float got = div_four_thirds_fast(g);
        if (got == 0.0f || std::signbit(got) != std::signbit(g)) fail("div_four_thirds_fast sign", b);
    }
    // with the signed-zero rule applied (adding -2^-149) the two forms agree for zeros as well
    if (mag == 0 && f2u(div_four_thirds_fast(g) + u2f(0x80000001u)) != f2u(want + u2f(0x80000001u))) fail("zero rule", b);
}

int main() {
    // every 1021st bit pattern (all exponents, both signs), plus every mantissa of a few binades
    for (uint64_t b = 0; b < (1ull << 32); b += 1021) check_division((uint32_t)b);
    const uint32_t binades[] = {0, 1, 22, 23, 24, 26, 27, 28, 100, 126, 127, 128, 200, 253, 254};
    for (uint32_t e : binades)
        for (uint32_t m = 0; m < (1u << 23); ++m) {
            check_division((e << 23) | m);
            check_division(0x80000000u | (e << 23) | m);
        }

    // bf16 round trip and round-to-nearest-even
    for (uint32_t h = 0; h < 65536; ++h) {
        const float f = bf16_to_f32((uint16_t)h);
        if (std::isnan(f)) continue;
        if (f32_to_bf16(f) != h) fail("bf16 round trip", h);
        const uint32_t base = h << 16;
        if ((h & 0x7f80u) == 0x7f80u || ((h + 1) & 0x7f80u) == 0x7f80u) continue;
        // just below / at / just above the midpoint to the next bf16 value
        if (f32_to_bf16(u2f(base + 0x7fffu)) != h) fail("bf16 below midpoint", h);
        if (f32_to_bf16(u2f(base + 0x8001u)) != h + 1) fail("bf16 above midpoint", h);
        if (f32_to_bf16(u2f(base + 0x8000u)) != ((h & 1u) ? h + 1 : h)) fail("bf16 tie to even", h);
    }

    // E2M1 grid, strict-threshold rounding, stochastic brackets
    const float grid[8] = {0.f, .5f, 1.f, 1.5f, 2.f, 3.f, 4.f, 6.f};
    for (int m = 0; m < 8; ++m) {
        if (e2m1_value(m) != grid[m]) fail("e2m1_value", (uint32_t)m);
        if (rtn_code(grid[m]) != m) fail("rtn grid point", (uint32_t)m);
        if (m < 7) {
            const float mid = 0.5f * (grid[m] + grid[m + 1]);
            if (rtn_code(mid) != m) fail("rtn tie goes down", (uint32_t)m);
            if (rtn_code(std::nextafter(mid, 10.f)) != m + 1) fail("rtn above tie goes up", (uint32_t)m);
            // up with probability p: up iff u < p, never at p = 0, always at p = 1 given u < 1
            const float a = grid[m] + 0.25f * (grid[m + 1] - grid[m]);
            if (sr_code(a, 0.2499f) != m + 1 || sr_code(a, 0.25f) != m) fail("sr threshold", (uint32_t)m);
            if (sr_code(grid[m + 1], 0.999f) != m + 1) fail("sr upper end", (uint32_t)m);
        }
    }
    if (rtn_code(1e9f) != 7 || sr_code(7.5f, 0.f) != 7) fail("saturation", 0);

    // the uniform of a 22-bit field f turns "u < p" into the carry out of floor(p 2^22) + f: every value of the top 16 bits
    // with the extreme and a few mixed low parts, p on and next to the boundary
    for (uint32_t hi = 0; hi < 65536; ++hi) {
        const uint32_t lows[5] = {0u, 1u, 32u, 62u, 63u};
        for (int li = 0; li < 5; ++li) {
            const uint32_t f = (hi << 6) | lows[li];
            const float u = uniform_from_field22(f);
            if (!(u > 0.0f && u < 1.0f)) fail("uniform_from_field22 range", f);
            const uint32_t boundary = 4194304u - f;  // smallest k with k + f >= 2^22
            for (int d = -2; d <= 2; ++d) {
                const int64_t k64 = (int64_t)boundary + d;
                if (k64 < 0 || k64 > 4194304) continue;
                const uint32_t k = (uint32_t)k64;  // p = k 2^-22, exact in fp32
                const float p = (float)k * (1.0f / 4194304.0f);
                if ((u < p) != (k + f >= 4194304u)) fail("uniform_from_field22", f);
                if (k < 4194304u) {
                    const float p_half = ((float)k + 0.5f) * (1.0f / 4194304.0f);  // p with bits below 2^-22
                    if ((u < p_half) != (k + f >= 4194304u)) fail("uniform_from_field22 (sub-grid p)", f);
                }
            }
        }
    }
    // an element's field: its word rotated left by a byte per position, top 22 bits
    {
        Philox4 ph;
        ph.w[0] = 0x04030201u; ph.w[1] = 0x08070605u; ph.w[2] = 0x0c0b0a09u; ph.w[3] = 0x100f0e0du;
        for (int j = 0; j < 16; ++j) {
            const uint32_t base = (uint32_t)(j & ~3) + 1u;  // value of the word's lowest byte
            uint32_t bytes[4];                               // most significant first after the rotation
            for (int i = 0; i < 4; ++i) bytes[i] = base + (uint32_t)((3 - (j & 3) - i + 8) & 3);
            const uint32_t rot = (bytes[0] << 24) | (bytes[1] << 16) | (bytes[2] << 8) | bytes[3];
            if (philox_field22(ph, j) != (rot >> 10)) fail("philox_field22", (uint32_t)j);
        }
    }

    // Philox4x32 known-answer vectors (Random123): 7 rounds, which the stream uses, and 10
    {
        const Philox4 a = philox4x32<10>(0, 0, 0, 0, 0, 0);
        const uint32_t wa[4] = {0x6627e8d5u, 0xe169c58du, 0xbc57ac4cu, 0x9b00dbd8u};
        const Philox4 b = philox4x32<10>(0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu);
        const uint32_t wb[4] = {0x408f276du, 0x41c83b0eu, 0xa20bc7c6u, 0x6d5451fdu};
        const Philox4 c = philox4x32<7>(0, 0, 0, 0, 0, 0);
        const uint32_t wc[4] = {0x5f6fb709u, 0x0d893f64u, 0x4f121f81u, 0x4f730a48u};
        const Philox4 d = philox4x32<7>(0x243f6a88u, 0x85a308d3u, 0x13198a2eu, 0x03707344u, 0xa4093822u, 0x299f31d0u);
        const uint32_t wd[4] = {0x4dfccabau, 0x190a87f0u, 0xc47362bau, 0xb6b5242au};
        const Philox4 e = philox_for_hexadecad(0, 0);
        for (int i = 0; i < 4; ++i) {
            if (a.w[i] != wa[i]) fail("philox-10 zeros", (uint32_t)i);
            if (b.w[i] != wb[i]) fail("philox-10 ones", (uint32_t)i);
            if (c.w[i] != wc[i]) fail("philox-7 zeros", (uint32_t)i);
            if (d.w[i] != wd[i]) fail("philox-7 pi", (uint32_t)i);
            if (e.w[i] != wc[i]) fail("the stream's call is the 7-round form", (uint32_t)i);
        }
    }

    // powers of two and the Hadamard constants
    for (int e = -149; e <= 127; ++e)
        if (pow2i(e) != std::ldexp(1.0f, e)) fail("pow2i", (uint32_t)(e + 149));
    if (hadamard_scale(32, BF16) != 0.1767578125f || hadamard_scale(64, BF16) != 0.125f ||
        hadamard_scale(128, BF16) != 0.08837890625f || hadamard_scale(32, F32) != (float)std::sqrt(1.0 / 32.0))
        fail("hadamard_scale", 0);

    // e^z with the fixed instruction sequence: within 1.5 ulp of the exact value wherever that is a normal number,
    // exact at 0, +inf above ln(FLT_MAX), and silu's limits; hashes over every bf16 input let the caller compare
    // bit for bit with another implementation of the same sequence
    uint64_t exp_hash = 1469598103934665603ull, silu_hash = 1469598103934665603ull;
    for (uint32_t h = 0; h < 65536; ++h) {
        const float z = bf16_to_f32((uint16_t)h);
        if (std::isnan(z)) continue;
        const float e = exp_fixed(z);
        exp_hash = (exp_hash ^ f2u(e)) * 1099511628211ull;
        silu_hash = (silu_hash ^ f2u(silu_fixed(z))) * 1099511628211ull;
        const double t = std::exp((double)z);
        if (t > 3.4028234663852886e38) { if (!(e == INFINITY || e > 3.3e38f)) fail("exp overflow", h); continue; }
        if (t < 1.1754943508222875e-38) { if (!(e >= 0.0f && e < 1.2e-38f)) fail("exp underflow", h); continue; }
        const double ulp = std::ldexp(1.0, std::ilogb(t) - 23);
        if (std::fabs((double)e - t) > 1.5 * ulp) fail("exp accuracy", h);
    }
    for (uint32_t i = 0; i < 2000000; ++i) {
        const float z = -104.0f + 193.0f * (float)i / 2000000.0f;
        const double t = std::exp((double)z);
        if (t > 3.4e38 || t < 1.2e-38) continue;
        if (std::fabs((double)exp_fixed(z) - t) > 1.5 * std::ldexp(1.0, std::ilogb(t) - 23)) fail("exp accuracy (sweep)", i);
    }
    if (exp_fixed(0.0f) != 1.0f || exp_fixed(89.0f) != INFINITY || exp_fixed(-200.0f) != 0.0f) fail("exp special values", 0);
    if (silu_fixed(0.0f) != 0.0f || silu_fixed(100.0f) != 100.0f || f2u(silu_fixed(-200.0f)) != 0x80000000u) fail("silu limits", 0);
    std::printf("exp_hash=%016llx silu_hash=%016llx\n", (unsigned long long)exp_hash, (unsigned long long)silu_hash);

    if (failures) {
        std::printf("%d failures\n", failures);
        return 1;
    }
    std::printf("ok\n");
    return 0;
}
