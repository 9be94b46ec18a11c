// Fast path of the fused block-Hadamard + MXFP4 quantizer ("group layout"): Hadamard block 32 for row-major,
// transposed and packed (re-quantize) input; Hadamard blocks 64 and 128 for row-major input.
//
// Same arithmetic as quantize.hip (the reference kernel
// src/models/quantization/quantizers/mxfp4_triton.py:19-174), different work decomposition: one lane
// owns a whole MX group of 32 values in registers, so
//   - the five butterfly stages, the group statistics and the scale are computed without any
//     cross-lane traffic and the per-group scalar work (sqrt, exponent extraction) is done once
//     instead of once per quarter group;
//   - the column sign of rotated element j is the same for every lane (j is a register index), so it
//     folds into the multiply by hd^-1/2;
//   - rounding, sign and nibble packing are done by gfx950's FP4 converts:
//       RTN  v_cvt_scalef32_pk_fp4_f32 is round-to-nearest-even; the reference rounds ties toward
//            zero, which differs exactly at .75, 1.75, 3.5.  Replacing the operand's bit pattern b by
//            (b - 1) | 1 moves every tie just below itself and nothing else across a boundary.
//       SR   v_cvt_scalef32_sr_pk_fp4_f32 rounds up iff floor(p * 2^22) + R >= 2^22 with p the position
//            inside the bracket and R = bits 31..10 of the random operand for the pair's first element,
//            bits 30..9 for its second (measured).  With R = the element's 22-bit field of the Philox stream this is
//            "u < p" for the uniform that stream defines (qm_math.h), bit for bit.  Each element gets its
//            own field (two converts per pair, merged with one mask).
//     The reference's sign rule "negative unless t > 0" makes +0 negative: adding -2^-149 first turns
//     both zeros into a negative denormal and changes no other value's code.
// Outputs are one 16-byte code store, one scale byte and one mask dword per lane, all contiguous across
// lanes; the input is read as 64 (bf16) or 128 (fp32) contiguous bytes per lane.
// The tiled row-major, transposed and re-quantizing kernels are written as jobs (qm_jobs.h) so that the whole-layer
// entry points can issue two of them in one grid.  rotate = false (row-major kernel only) skips the butterfly: the
// caller has already applied a dense rotation.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "qm_jobs.h"
#include "qm_kernels.h"
#include "qm_math.h"

namespace qm {

namespace {

typedef float v2f __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void butterfly32(float (&v)[32]) {
#pragma unroll
    for (int h = 1; h < 32; h <<= 1) {
#pragma unroll
        for (int i = 0; i < 32; ++i) {
            if (i & h) continue;
            const float a = v[i], b = v[i + h];
            v[i] = a + b;
            v[i + h] = a - b;
        }
    }
}

// pairwise tree: adjacent pairs, then pairs of pairs, ... (the canonical order of the group sums)
__device__ __forceinline__ float tree_sum32(const float (&p)[32]) {
    float t[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) t[i] = p[2 * i] + p[2 * i + 1];
#pragma unroll
    for (int n = 8; n >= 1; n >>= 1)
#pragma unroll
        for (int i = 0; i < n; ++i) t[i] = t[2 * i] + t[2 * i + 1];
    return t[0];
}

struct GroupCodes {
    uint32_t w[4];        // 32 nibbles, element i in bits [4(i%8), +4) of word i/8
    uint32_t scale_byte;  // E8M0
    uint32_t keep;        // bit i = |t_i| < 6
    float deq_scale;      // what a code value is multiplied by in the de-quantized tensor
};

#define kNegTiny (u2f(0x80000001u))  // -2^-149

// v_cvt_scalef32_sr_pk_fp4_f32 replaces byte SEL of its destination and keeps the other three, but the
// compiler builtin of this toolchain does not tie the destination to its `old` operand (the untouched bytes
// come back as whatever the allocated register held), so the instruction is issued directly.
template <int SEL>
__device__ __forceinline__ void sr_convert_pair(uint32_t& dst, v2f pair, uint32_t rnd, float scale) {
    if constexpr (SEL == 0) asm("v_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, %3" : "+v"(dst) : "v"(pair), "v"(rnd), "v"(scale));
    else if constexpr (SEL == 1) asm("v_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, %3 op_sel:[0,0,1,0]" : "+v"(dst) : "v"(pair), "v"(rnd), "v"(scale));
    else if constexpr (SEL == 2) asm("v_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, %3 op_sel:[0,0,0,1]" : "+v"(dst) : "v"(pair), "v"(rnd), "v"(scale));
    else asm("v_cvt_scalef32_sr_pk_fp4_f32 %0, %1, %2, %3 op_sel:[0,0,1,1]" : "+v"(dst) : "v"(pair), "v"(rnd), "v"(scale));
}

// ties-toward-zero via the round-to-nearest-even convert (see the file comment)
__device__ __forceinline__ float tie_nudge(float v) {
    return u2f(__builtin_elementwise_sub_sat(f2u(v), 1u) | 1u);
}

template <int MODE, bool WANT_MASK>
__device__ __forceinline__ void quantize_group_regs(const float (&g)[32], uint64_t seed, int64_t group_index,
                                                    GroupCodes& o) {
    constexpr bool kQuest = (MODE == QUEST_RTN || MODE == QUEST_SR);
    constexpr bool kSR = (MODE == ABSMAX_SR || MODE == QUEST_SR);
    float hw_scale;   // power of two the convert divides by
    uint32_t thr_bits;  // bit pattern of 6 * scale: |g| < thr  <=>  |t| < 6
    float t[32];
    bool all_zero = false;
    if constexpr (kQuest) {
        float sq[32];
#pragma unroll
        for (int i = 0; i < 32; ++i) sq[i] = g[i] * g[i];
        const float ms = tree_sum32(sq) * 0.03125f;
        const float m = tree_sum32(g) * 0.03125f;
        const float mm = m * m;
        float var = ms - mm;
        var = var > 0.0f ? var : 0.0f;
        const float sd = __builtin_sqrtf(var);
        const float gs = kQuestG * sd;
        const float s = gs + 1e-8f;
        int E = (int)((f2u(s) >> 23) & 0xffu) - 127;
        E = E > 127 ? 127 : E;
        o.scale_byte = (uint32_t)(E + 127);
        hw_scale = pow2i(E);
        o.deq_scale = hw_scale;
        thr_bits = f2u(6.0f * hw_scale);
#pragma unroll
        for (int i = 0; i < 32; ++i) t[i] = g[i];
    } else {
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < 32; ++i) a = fmaxf(a, fabsf(g[i]));
        all_zero = (a == 0.0f);
        int k = (int)((f2u(a) >> 23) & 0xffu) - 129;
        k = k < -127 ? -127 : (k > 127 ? 127 : k);
        o.scale_byte = (uint32_t)(k + 127);
        hw_scale = pow2i(k);
        o.deq_scale = scale_pow2(kFourThirds, k);
        // |t| < 6 with t = RN(g 2^-k / d): evaluated on the quotient h = RN(g / d) against 6 * 2^k
        thr_bits = f2u(6.0f * hw_scale);
        // t = RN(RN(g 2^-k) / d) by definition.  For a group whose maximum is at least 2^-60 this is RN(g / d) scaled by
        // 2^-k inside the convert: the two-operation quotient is exact for |g| >= 2^-100, and a smaller element lies
        // below 2^-38 of the scale, so its code is a zero whose sign is the element's own whatever the quotient's last
        // bit.  A group with a smaller non-zero maximum (where g / d would lose bits to underflow) follows the
        // definition literally, with a true division, and hands the convert an already scaled value.
        if (__builtin_expect(a < 0x1p-60f && !all_zero, 0)) {
#pragma unroll
            for (int i = 0; i < 32; ++i) t[i] = scale_pow2(g[i], -k) / kFourThirds;
            hw_scale = 1.0f;
            thr_bits = f2u(6.0f);
        } else {
#pragma unroll
            for (int i = 0; i < 32; ++i) t[i] = div_four_thirds_fast(g[i]);
        }
    }
    o.keep = 0u;
    if constexpr (WANT_MASK) {
        // clip mask, most significant element first so that element 0 lands in bit 0
        // one compare into the carry flag and one add-with-carry (keep = 2 keep + flag) per element, sixteen
        // elements per statement (the operand limit of an asm statement)
        uint32_t keep = 0u;
        const float thr = u2f(thr_bits);
#define QM_KEEP_BIT(N) "v_cmp_lt_f32_e64 vcc, |%" #N "|, %17\n\tv_addc_co_u32_e32 %0, vcc, %0, %0, vcc\n\t"
#define QM_KEEP_16(B)                                                                                               \
    asm(QM_KEEP_BIT(16) QM_KEEP_BIT(15) QM_KEEP_BIT(14) QM_KEEP_BIT(13) QM_KEEP_BIT(12) QM_KEEP_BIT(11) QM_KEEP_BIT(10) \
        QM_KEEP_BIT(9) QM_KEEP_BIT(8) QM_KEEP_BIT(7) QM_KEEP_BIT(6) QM_KEEP_BIT(5) QM_KEEP_BIT(4) QM_KEEP_BIT(3)        \
        QM_KEEP_BIT(2) QM_KEEP_BIT(1)                                                                                   \
        : "+v"(keep)                                                                                                    \
        : "v"(t[(B)]), "v"(t[(B) + 1]), "v"(t[(B) + 2]), "v"(t[(B) + 3]), "v"(t[(B) + 4]), "v"(t[(B) + 5]),             \
          "v"(t[(B) + 6]), "v"(t[(B) + 7]), "v"(t[(B) + 8]), "v"(t[(B) + 9]), "v"(t[(B) + 10]), "v"(t[(B) + 11]),       \
          "v"(t[(B) + 12]), "v"(t[(B) + 13]), "v"(t[(B) + 14]), "v"(t[(B) + 15]), "v"(thr)                              \
        : "vcc")
        QM_KEEP_16(16);
        QM_KEEP_16(0);
#undef QM_KEEP_16
#undef QM_KEEP_BIT
        o.keep = all_zero ? 0u : keep;
    }

    // the converts' byte selector must be a literal, hence the macros
#define QM_RTN_PAIR(B)                                                                                   \
    w = __builtin_amdgcn_cvt_scalef32_pk_fp4_f32(w, tie_nudge(t[wi * 8 + 2 * (B)] + kNegTiny),           \
                                                 tie_nudge(t[wi * 8 + 2 * (B) + 1] + kNegTiny), hw_scale, (B));
    // element j of a Philox call (16 elements): its random field is the top 22 bits of word j/4 rotated left by
    // 8 * (j%4).  The convert reads the field of a pair's first element from bits 31..10 of its random operand and that of
    // the second from bits 30..9, so the even element's operand is the word rotated by 0 or 16 bits and the odd element's
    // the word rotated by 7 or 23 (one more bit to the right): one v_alignbit_b32 each, none for a word's first element.
#define QM_SR_PAIR(B, J0)                                                                                 \
    {                                                                                                     \
        const uint32_t pw = ph.w[(J0) >> 2];                                                              \
        const uint32_t r_even = ((J0) & 3) == 0 ? pw : __builtin_amdgcn_alignbit(pw, pw, 16);             \
        const uint32_t r_odd = __builtin_amdgcn_alignbit(pw, pw, ((J0) & 3) == 0 ? 25 : 9);               \
        const v2f pr = {t[wi * 8 + 2 * (B)] + kNegTiny, t[wi * 8 + 2 * (B) + 1] + kNegTiny};              \
        sr_convert_pair<(B)>(even, pr, r_even, hw_scale);                                                 \
        sr_convert_pair<(B)>(odd, pr, r_odd, hw_scale);                                                   \
    }
    if constexpr (!kSR) {
#pragma unroll
        for (int wi = 0; wi < 4; ++wi) {
            uint32_t w = 0u;
            QM_RTN_PAIR(0) QM_RTN_PAIR(1) QM_RTN_PAIR(2) QM_RTN_PAIR(3)
            o.w[wi] = w;
        }
    } else {
        Philox4 ph;
#pragma unroll
        for (int wi = 0; wi < 4; ++wi) {
            // words 0,1 of the call serve the even octet of the pair, words 2,3 the odd one
            if ((wi & 1) == 0) ph = philox_for_hexadecad(seed, (uint64_t)(group_index * 2 + (wi >> 1)));
            uint32_t even = 0u, odd = 0u;  // converts driven by the even / odd element's random byte
            if ((wi & 1) == 0) { QM_SR_PAIR(0, 0) QM_SR_PAIR(1, 2) QM_SR_PAIR(2, 4) QM_SR_PAIR(3, 6) }
            else { QM_SR_PAIR(0, 8) QM_SR_PAIR(1, 10) QM_SR_PAIR(2, 12) QM_SR_PAIR(3, 14) }
            o.w[wi] = (even & 0x0f0f0f0fu) | (odd & 0xf0f0f0f0u);
        }
    }
#undef QM_RTN_PAIR
#undef QM_SR_PAIR
}

template <typename T>
__device__ __forceinline__ void load_group(const T* __restrict__ p, float (&v)[32]) {
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint4 raw = reinterpret_cast<const uint4*>(p)[q];
            const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[q * 8 + 2 * i] = u2f(w[i] << 16);
                v[q * 8 + 2 * i + 1] = u2f(w[i] & 0xffff0000u);
            }
        }
    } else {
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const float4 f = reinterpret_cast<const float4*>(p)[q];
            v[q * 4] = f.x; v[q * 4 + 1] = f.y; v[q * 4 + 2] = f.z; v[q * 4 + 3] = f.w;
        }
    }
}

template <typename T>
__device__ __forceinline__ void store_dequant(T* __restrict__ p, const GroupCodes& o) {
    float v[32];
#pragma unroll
    for (int i = 0; i < 32; ++i) {
        const uint32_t nib = (o.w[i >> 3] >> (4 * (i & 7))) & 15u;
        const float q = e2m1_value((int)(nib & 7u));
        v[i] = ((nib & 8u) ? -q : q) * o.deq_scale;
    }
    if constexpr (sizeof(T) == 2) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i)
                w[i] = (uint32_t)f32_to_bf16(v[q * 8 + 2 * i]) | ((uint32_t)f32_to_bf16(v[q * 8 + 2 * i + 1]) << 16);
            reinterpret_cast<uint4*>(p)[q] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    } else {
#pragma unroll
        for (int q = 0; q < 8; ++q)
            reinterpret_cast<float4*>(p)[q] = make_float4(v[q * 4], v[q * 4 + 1], v[q * 4 + 2], v[q * 4 + 3]);
    }
}

struct GroupOut {
    uint4* codes;        // [n_groups]
    uint8_t* scales;     // [n_groups]
    uint32_t* maskbits;  // [n_groups] or null
    void* dequant;       // [n_groups * 32] of T or null
};

// x @ H for one chunk of 32: butterfly, then hd^-1/2 with the column sign folded in (wave-uniform)
__device__ __forceinline__ void rotate_group(float (&v)[32], float c, uint32_t sign_word, bool rotate = true) {
    if (rotate) butterfly32(v);  // uniform; without it (c = 1, no signs) the group passes through unchanged
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        const float cj = u2f(f2u(c) ^ (((sign_word >> j) & 1u) << 31));  // wave-uniform: stays in scalar registers
        v[j] = v[j] * cj;
    }
}

// ---- dense 32x32 rotation (rerotate="O32", quantizers/mxfp4.py:61-64 of the reference) on the matrix pipe ----------
// The reference applies the matrix with tl.dot inside its kernel (mxfp4_triton.py:44-45).  Here each lane owns one
// group of 32 values; v_mfma_f32_32x32x2_f32 computes D[j][n] += H[k][j] x[n][k] for 32 groups n at a time, and sixteen
// chained instructions walk k = 0..31.  The instruction evaluates acc = fma(a, b, acc) per term in ascending k
// (measured against every candidate order on random fp32 data: no mismatch), which is the order the test oracle states.
// Lanes 0..31 hold groups "lo", lanes 32..63 groups "hi": v_permlane32_swap deals a lane's pair (k, k+1) out as the two
// k rows the instruction wants from the two half-waves, and collects the results (a lane gets the 16 rotated values of
// its group that the other half-wave computed).  Every lane of the wave must be active.
typedef float v16f __attribute__((ext_vector_type(16)));
struct DenseFrag {
    float a[16];  // H[2t + lane/32][lane%32], t = 0..15, rounded to the tensor's dtype
};
__device__ __forceinline__ void load_dense_frag(const float* __restrict__ matrix, int dtype, DenseFrag& f) {
    const int lane = threadIdx.x & 63, j = lane & 31, half = lane >> 5;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        float h = matrix[(2 * t + half) * 32 + j];
        if (dtype == BF16) h = bf16_to_f32(f32_to_bf16(h));
        f.a[t] = h;
    }
}
__device__ __forceinline__ void dense_rotate(float (&v)[32], const DenseFrag& f) {
    v16f lo, hi;
#pragma unroll
    for (int e = 0; e < 16; ++e) lo[e] = hi[e] = 0.0f;
#pragma unroll
    for (int t = 0; t < 16; ++t) {
        // after the swap: first = (k = 2t of groups lo | k = 2t+1 of groups lo), second = the same of groups hi
        const auto r = __builtin_amdgcn_permlane32_swap(f2u(v[2 * t]), f2u(v[2 * t + 1]), false, false);
        lo = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[t], u2f(r[0]), lo, 0, 0, 0);
        hi = __builtin_amdgcn_mfma_f32_32x32x2f32(f.a[t], u2f(r[1]), hi, 0, 0, 0);
    }
    // accumulator element e of a lane is output row j = 8 (e / 4) + 4 (lane / 32) + e % 4 of group lane % 32
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        const auto r = __builtin_amdgcn_permlane32_swap(f2u(lo[e]), f2u(hi[e]), false, false);
        v[8 * (e / 4) + (e % 4)] = u2f(r[0]);
        v[8 * (e / 4) + 4 + (e % 4)] = u2f(r[1]);
    }
}

// rotate (hd = 32) + quantize the group in v; gi is its logical (row-major) group index, which also keys the
// random stream; ci is the index of its 16 code bytes in the code buffer (= gi for row-major codes)
template <typename T, int MODE, bool WANT_MASK>
__device__ __forceinline__ void finish_group(float (&v)[32], int64_t gi, int64_t ci, float c, uint32_t sign_word,
                                             uint64_t seed, const GroupOut& out, bool rotate) {
    rotate_group(v, c, sign_word, rotate);
    GroupCodes o;
    quantize_group_regs<MODE, WANT_MASK>(v, seed, gi, o);
    out.codes[ci] = make_uint4(o.w[0], o.w[1], o.w[2], o.w[3]);
    out.scales[gi] = (uint8_t)o.scale_byte;
    if constexpr (WANT_MASK) out.maskbits[gi] = o.keep;
    if (out.dequant) store_dequant<T>(reinterpret_cast<T*>(out.dequant) + gi * 32, o);
}

template <typename T, int MODE, bool WANT_MASK>
__global__ __launch_bounds__(256) void quantize_rowmajor_g32_kernel(const T* __restrict__ x, int64_t n_groups, float c,
                                                                    uint32_t sign_word, uint64_t seed, GroupOut out,
                                                                    int rotate) {
    job_starts();
    const int64_t gi = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (gi >= n_groups) return;
    float v[32];
    load_group<T>(x + gi * 32, v);
    job_requests_issued();
    finish_group<T, MODE, WANT_MASK>(v, gi, gi, c, sign_word, seed, out, rotate != 0);
}

// Row-major input with a dense rotation: one group per lane, flat over the tensor; row-major or tiled code bytes.
template <typename T, int MODE, bool WANT_MASK>
__global__ __launch_bounds__(256) void quantize_rowmajor_dense_kernel(const T* __restrict__ x, int64_t n_groups, int groups_per_row,
                                                                      const float* __restrict__ matrix, uint64_t seed,
                                                                      GroupOut out, int tiled) {
    const int64_t gi = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool valid = gi < n_groups;
    DenseFrag frag;
    load_dense_frag(matrix, sizeof(T) == 2 ? BF16 : F32, frag);
    float v[32];
    if (valid) {
        load_group<T>(x + gi * 32, v);
    } else {
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = 0.0f;
    }
    dense_rotate(v, frag);  // the whole wave, also past the end of the tensor
    if (!valid) return;
    GroupCodes o;
    quantize_group_regs<MODE, WANT_MASK>(v, seed, gi, o);
    int64_t ci = gi;
    if (tiled) {
        const int64_t row = gi / groups_per_row;
        const int g = (int)(gi - row * groups_per_row);
        ci = (row >> 4) * 16 * groups_per_row + ((g >> 2) * 64 + (int)(row & 15) * 4 + (g & 3));
    }
    out.codes[ci] = make_uint4(o.w[0], o.w[1], o.w[2], o.w[3]);
    out.scales[gi] = (uint8_t)o.scale_byte;
    if constexpr (WANT_MASK) out.maskbits[gi] = o.keep;
    if (out.dequant) store_dequant<T>(reinterpret_cast<T*>(out.dequant) + gi * 32, o);
}

template <typename T, bool WANT_MASK>
void launch_rowmajor_dense(int mode, const void* x, int64_t rows, int64_t cols, const float* matrix, uint64_t seed,
                           const GroupOut& out, bool tiled, hipStream_t stream) {
    const T* xp = reinterpret_cast<const T*>(x);
    const int64_t n_groups = rows * cols / 32;
    const int gpr = (int)(cols / 32);
    dim3 grid((unsigned)((n_groups + 255) / 256)), block(256);
    switch (mode) {
        case QUEST_RTN: quantize_rowmajor_dense_kernel<T, QUEST_RTN, WANT_MASK><<<grid, block, 0, stream>>>(xp, n_groups, gpr, matrix, seed, out, (int)tiled); break;
        case ABSMAX_RTN: quantize_rowmajor_dense_kernel<T, ABSMAX_RTN, WANT_MASK><<<grid, block, 0, stream>>>(xp, n_groups, gpr, matrix, seed, out, (int)tiled); break;
        case ABSMAX_SR: quantize_rowmajor_dense_kernel<T, ABSMAX_SR, WANT_MASK><<<grid, block, 0, stream>>>(xp, n_groups, gpr, matrix, seed, out, (int)tiled); break;
        default: quantize_rowmajor_dense_kernel<T, QUEST_SR, WANT_MASK><<<grid, block, 0, stream>>>(xp, n_groups, gpr, matrix, seed, out, (int)tiled); break;
    }
}

// Tiled code layout ([rows/16][cols/128][16 rows][64 bytes]).  Workgroup b owns block b / chunks of 16 rows and run
// b % chunks of 512 columns (four code tiles); wave w owns rows 4w..4w+3 of the block, lane l its row l / 16 and
// group l % 16 of the run: the wave reads four contiguous KiB (bf16) and writes, per tile, four rows' 64-byte pieces
// = 256 contiguous bytes.  The four scale bytes of four adjacent groups are gathered into one dword store.
template <typename T, int MODE, bool WANT_MASK>
struct RowmajorTiledJob {
    const T* x;
    int64_t cols;
    int chunks;
    float c;
    uint32_t sign_word;
    uint64_t seed;
    const uint64_t* seed_base = nullptr;  // device memory, or null: a value the kernel adds to `seed` when it runs
    GroupOut out;
    unsigned blocks;

    RowmajorTiledJob(const void* x_, int64_t rows, int64_t cols_, float c_, uint32_t sign_word_, uint64_t seed_,
                     const GroupOut& out_)
        : x(reinterpret_cast<const T*>(x_)), cols(cols_), chunks((int)((cols_ / 128 + 3) / 4)), c(c_),
          sign_word(sign_word_), seed(seed_), out(out_), blocks((unsigned)((rows / 16) * ((cols_ / 128 + 3) / 4))) {}

    __device__ __forceinline__ void run(unsigned bid) const {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int groups = (int)(cols / 32);  // per row
        const unsigned rb = bid / (unsigned)chunks;
        const int g = (int)(bid - rb * chunks) * 16 + (lane & 15);  // group within the row
        if (g >= groups) return;  // cols % 128 == 0: quads of lanes leave together, the gather below sees full quads
        const int rin = wave * 4 + (lane >> 4);  // row within the block
        // uniform 64-bit block bases + small per-lane offsets
        const int64_t gi = (int64_t)rb * 16 * groups + (rin * groups + g);
        const int64_t ci = (int64_t)rb * 16 * groups + ((g >> 2) * 64 + rin * 4 + (g & 3));
        float v[32];
        load_group<T>(x + gi * 32, v);
        job_requests_issued();
        rotate_group(v, c, sign_word);
        GroupCodes o;
        quantize_group_regs<MODE, WANT_MASK>(v, seed_base ? seed + *seed_base : seed, gi, o);
        job_stores_next();
        out.codes[ci] = make_uint4(o.w[0], o.w[1], o.w[2], o.w[3]);
        // quad_perm broadcasts of lanes 1, 2, 3 of each quad
        const uint32_t s1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)o.scale_byte, 0x55, 0xf, 0xf, false);
        const uint32_t s2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)o.scale_byte, 0xAA, 0xf, 0xf, false);
        const uint32_t s3 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)o.scale_byte, 0xFF, 0xf, 0xf, false);
        if ((lane & 3) == 0)
            *reinterpret_cast<uint32_t*>(out.scales + gi) = o.scale_byte | (s1 << 8) | (s2 << 16) | (s3 << 24);
        if constexpr (WANT_MASK) out.maskbits[gi] = o.keep;
        if (out.dequant) store_dequant<T>(reinterpret_cast<T*>(out.dequant) + gi * 32, o);
    }
};

template <typename T, bool WANT_MASK>
void launch_rowmajor_g32(int mode, const void* x, int64_t rows, int64_t cols, bool tiled, float c, uint32_t sign_word,
                         uint64_t seed, const GroupOut& out, bool rotate, hipStream_t stream) {
    const T* xp = reinterpret_cast<const T*>(x);
    if (tiled) {
        const auto go = [&](auto job) { launch_job(job, stream); };
        switch (mode) {
            case QUEST_RTN: go(RowmajorTiledJob<T, QUEST_RTN, WANT_MASK>(x, rows, cols, c, sign_word, seed, out)); break;
            case ABSMAX_RTN: go(RowmajorTiledJob<T, ABSMAX_RTN, WANT_MASK>(x, rows, cols, c, sign_word, seed, out)); break;
            case ABSMAX_SR: go(RowmajorTiledJob<T, ABSMAX_SR, WANT_MASK>(x, rows, cols, c, sign_word, seed, out)); break;
            default: go(RowmajorTiledJob<T, QUEST_SR, WANT_MASK>(x, rows, cols, c, sign_word, seed, out)); break;
        }
        return;
    }
    const int64_t n_groups = rows * cols / 32;
    dim3 grid((unsigned)((n_groups + 255) / 256)), block(256);
    switch (mode) {
        case QUEST_RTN: quantize_rowmajor_g32_kernel<T, QUEST_RTN, WANT_MASK><<<grid, block, 0, stream>>>(xp, n_groups, c, sign_word, seed, out, (int)rotate); break;
        case ABSMAX_RTN: quantize_rowmajor_g32_kernel<T, ABSMAX_RTN, WANT_MASK><<<grid, block, 0, stream>>>(xp, n_groups, c, sign_word, seed, out, (int)rotate); break;
        case ABSMAX_SR: quantize_rowmajor_g32_kernel<T, ABSMAX_SR, WANT_MASK><<<grid, block, 0, stream>>>(xp, n_groups, c, sign_word, seed, out, (int)rotate); break;
        default: quantize_rowmajor_g32_kernel<T, QUEST_SR, WANT_MASK><<<grid, block, 0, stream>>>(xp, n_groups, c, sign_word, seed, out, (int)rotate); break;
    }
}

// ---- Hadamard blocks 64 and 128, row-major ---------------------------------------------------------------
// Same one-group-per-lane layout; a Hadamard chunk is HD/32 consecutive lanes (a lane pair or a quad).  The
// five in-register stages are followed by the stride-32 (and stride-64) stages across the lanes of the chunk, one
// DPP-fed multiply-add per element: own + partner in the lower lane of a butterfly, own - partner in the upper one.
// The upper lane's exact value is partner - own = -(own - partner): rounding is symmetric, so the negation commutes
// with it, and it is folded into the column sign applied at the end (a lane's values are negated once per stage in
// which it is the upper lane).  The column signs differ per lane of the chunk; they are applied as lane masks held in
// scalar registers (bit l of mask j: negate element j in lane l), one select per element.
template <int CTRL>
__device__ __forceinline__ void cross_lane_stage(float (&v)[32], float s) {
    // s = +1 in the lower lane, -1 in the upper one.  An instruction reads its own destination register from the
    // partner lane; the leading s_nop keeps the two wait states a DPP read needs after a vector write to that register
    // (the compiler does not look into assembly statements).
#define QM_X(N) "v_fmac_f32_dpp %" #N ", %" #N ", %16 quad_perm:[%17,%18,%19,%20] row_mask:0xf bank_mask:0xf bound_ctrl:1\n\t"
#define QM_STAGE16(B)                                                                                                   \
    asm volatile("s_nop 1\n\t" QM_X(0) QM_X(1) QM_X(2) QM_X(3) QM_X(4) QM_X(5) QM_X(6) QM_X(7) QM_X(8) QM_X(9) QM_X(10) QM_X(11)  \
                 QM_X(12) QM_X(13) QM_X(14) QM_X(15)                                                                     \
                 : "+v"(v[(B)]), "+v"(v[(B) + 1]), "+v"(v[(B) + 2]), "+v"(v[(B) + 3]), "+v"(v[(B) + 4]), "+v"(v[(B) + 5]),  \
                   "+v"(v[(B) + 6]), "+v"(v[(B) + 7]), "+v"(v[(B) + 8]), "+v"(v[(B) + 9]), "+v"(v[(B) + 10]),             \
                   "+v"(v[(B) + 11]), "+v"(v[(B) + 12]), "+v"(v[(B) + 13]), "+v"(v[(B) + 14]), "+v"(v[(B) + 15])          \
                 : "v"(s), "n"(CTRL & 3), "n"((CTRL >> 2) & 3), "n"((CTRL >> 4) & 3), "n"((CTRL >> 6) & 3))
    QM_STAGE16(0);
    QM_STAGE16(16);
#undef QM_STAGE16
#undef QM_X
}

template <typename T, int MODE, bool WANT_MASK, int HD>
__global__ __launch_bounds__(256) void quantize_rowmajor_wide_kernel(const T* __restrict__ x, int64_t n_groups, float c,
                                                                     SignBits sf, uint64_t seed, GroupOut out) {
    static_assert(HD == 64 || HD == 128, "lane pairs or quads");
    job_starts();
    const int64_t gi = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (gi >= n_groups) return;  // n_groups is a multiple of HD/32: the lanes of a chunk leave together
    float v[32];
    load_group<T>(x + gi * 32, v);
    job_requests_issued();
    butterfly32(v);
    const int part = (int)threadIdx.x & (HD / 32 - 1);
    cross_lane_stage<0xB1>(v, (part & 1) ? -1.0f : 1.0f);                           // quad_perm [1,0,3,2]: stride 32
    if constexpr (HD == 128) cross_lane_stage<0x4E>(v, (part & 2) ? -1.0f : 1.0f);  // quad_perm [2,3,0,1]: stride 64
    // sf holds, per element j, a field of HD/32 bits: bit p = negate element j in the chunk's lane p (column sign
    // xor the stage negations above).  field * 0x5555... (or 0x1111...) spreads it over the wave's chunks.
    constexpr int P = HD / 32;
    constexpr uint32_t kUnit = P == 2 ? 0x55555555u : 0x11111111u;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
        const uint32_t field = (sf.w[(j * P) >> 5] >> ((j * P) & 31)) & ((1u << P) - 1u);  // wave-uniform: scalar registers
        const uint32_t half = field * kUnit;
        const uint64_t m = ((uint64_t)half << 32) | half;
        const float scaled = v[j] * c;
        asm("v_cndmask_b32_e64 %0, %1, -%1, %2" : "=v"(v[j]) : "v"(scaled), "s"(m));
    }
    GroupCodes o;
    quantize_group_regs<MODE, WANT_MASK>(v, seed, gi, o);
    job_stores_next();
    out.codes[gi] = make_uint4(o.w[0], o.w[1], o.w[2], o.w[3]);
    out.scales[gi] = (uint8_t)o.scale_byte;
    if constexpr (WANT_MASK) out.maskbits[gi] = o.keep;
    if (out.dequant) store_dequant<T>(reinterpret_cast<T*>(out.dequant) + gi * 32, o);
}

// Per-element negation fields of the wide kernel: bit p of field j = column sign of rotated element 32 p + j, xor 1 for
// the lanes of a chunk whose index has an odd number of set bits (their values come out of the cross-lane stages negated).
template <int HD>
SignBits wide_sign_fields(const SignBits& sb) {
    constexpr int P = HD / 32;
    SignBits sf{{0u, 0u, 0u, 0u}};
    for (int j = 0; j < 32; ++j) {
        uint32_t field = 0u;
        for (int p = 0; p < P; ++p) field |= (((sb.w[p] >> j) & 1u) ^ (uint32_t)(__builtin_popcount((unsigned)p) & 1)) << p;
        sf.w[(j * P) >> 5] |= field << ((j * P) & 31);
    }
    return sf;
}

template <typename T, bool WANT_MASK, int HD>
void launch_rowmajor_wide(int mode, const void* x, int64_t n, float c, const SignBits& sb, uint64_t seed,
                          const GroupOut& out, hipStream_t stream) {
    const T* xp = reinterpret_cast<const T*>(x);
    const int64_t n_groups = n / 32;
    const SignBits sf = wide_sign_fields<HD>(sb);
    dim3 grid((unsigned)((n_groups + 255) / 256)), block(256);
    switch (mode) {
        case QUEST_RTN: quantize_rowmajor_wide_kernel<T, QUEST_RTN, WANT_MASK, HD><<<grid, block, 0, stream>>>(xp, n_groups, c, sf, seed, out); break;
        case ABSMAX_RTN: quantize_rowmajor_wide_kernel<T, ABSMAX_RTN, WANT_MASK, HD><<<grid, block, 0, stream>>>(xp, n_groups, c, sf, seed, out); break;
        case ABSMAX_SR: quantize_rowmajor_wide_kernel<T, ABSMAX_SR, WANT_MASK, HD><<<grid, block, 0, stream>>>(xp, n_groups, c, sf, seed, out); break;
        default: quantize_rowmajor_wide_kernel<T, QUEST_SR, WANT_MASK, HD><<<grid, block, 0, stream>>>(xp, n_groups, c, sf, seed, out); break;
    }
}

// ---- transposed input: x is [P, Q] row-major, output is the [Q, P] tensor quantized along P ----------
// A workgroup owns a strip of 256 bytes of columns (128 bf16 / 64 fp32) by 128 rows; wave w owns p-group w.
// A lane reads its column (bf16: two adjacent columns per 32-bit load) at 32 successive rows straight from
// global memory: each wave load is one contiguous 256-byte row segment, 8 KiB in flight per wave, no LDS and
// no barrier on the input side.  Codes and scales go through LDS so that each q row leaves the workgroup as
// one contiguous 64-byte (codes) / 4-byte (scales) piece.
template <typename T>
struct TrTile {
    static constexpr int kQ = 256 / (int)sizeof(T);      // 128 columns of bf16, 64 of fp32
    static constexpr int kGroupsPerLane = kQ / 64;       // 2 for bf16, 1 for fp32
};
constexpr int kTrP = 128;

template <typename T, int MODE, bool DENSE = false>
struct TransposedJob {
    const T* x;
    int64_t P, Q;
    float c;
    uint32_t sign_word;
    uint64_t seed;
    const uint64_t* seed_base = nullptr;  // device memory, or null: a value the kernel adds to `seed` when it runs
    uint8_t* codes;
    uint8_t* scales;
    void* dequant;
    bool tiled_out;
    const float* matrix;  // DENSE: the rotation, [32][32] fp32 (c and sign_word are then unused)
    unsigned grid_p, blocks;

    TransposedJob(const void* x_, int64_t P_, int64_t Q_, float c_, uint32_t sign_word_, uint64_t seed_, uint8_t* codes_,
                  uint8_t* scales_, void* dequant_, bool tiled_out_, const float* matrix_ = nullptr)
        : x(reinterpret_cast<const T*>(x_)), P(P_), Q(Q_), c(c_), sign_word(sign_word_), seed(seed_), codes(codes_),
          scales(scales_), dequant(dequant_), tiled_out(tiled_out_), matrix(matrix_), grid_p((unsigned)((P_ + kTrP - 1) / kTrP)),
          blocks((unsigned)(((P_ + kTrP - 1) / kTrP) * ((Q_ + TrTile<T>::kQ - 1) / TrTile<T>::kQ))) {}

    __device__ __forceinline__ void run(unsigned bid) const {
        constexpr int TQ = TrTile<T>::kQ;
        constexpr int GPL = TrTile<T>::kGroupsPerLane;
        __shared__ uint4 ocodes[TQ * 4];      // [q][4 groups x 16 B]
        __shared__ uint32_t oscales[TQ];      // [q][4 B]
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // tells the compiler it is wave-uniform
        const unsigned bq = bid / grid_p;
        const int64_t p0 = (int64_t)(bid - bq * grid_p) * kTrP, q0 = (int64_t)bq * TQ;
        const int64_t pbase = p0 + wave * 32;       // this wave's group along p
        const int64_t qa = q0 + lane * GPL;         // this lane's first column
        const bool active = pbase < P && qa < Q;    // P % 32 == 0 and Q % 8 == 0: all of a lane's groups or none
        float v[GPL][32];
        if (active) {
            // uniform row pointers (scalar unit) + the lane's 32-bit dword offset: no per-lane 64-bit address math
            const uint32_t* row = reinterpret_cast<const uint32_t*>(x + pbase * Q + q0);
            const int64_t row_dw = Q * (int64_t)sizeof(T) / 4;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                const uint32_t w = (row + i * row_dw)[(uint32_t)lane];
                if constexpr (sizeof(T) == 2) {
                    v[0][i] = u2f(w << 16);
                    v[1][i] = u2f(w & 0xffff0000u);
                } else {
                    v[0][i] = u2f(w);
                }
            }
        } else if constexpr (DENSE) {
#pragma unroll
            for (int gq = 0; gq < GPL; ++gq)
#pragma unroll
                for (int i = 0; i < 32; ++i) v[gq][i] = 0.0f;
        }
        job_requests_issued();
        if constexpr (DENSE) {  // the matrix instruction needs the whole wave, lanes outside the tensor included
            DenseFrag frag;
            load_dense_frag(matrix, sizeof(T) == 2 ? BF16 : F32, frag);
#pragma unroll
            for (int gq = 0; gq < GPL; ++gq) dense_rotate(v[gq], frag);
        }
        if (active) {
#pragma unroll
            for (int gq = 0; gq < GPL; ++gq) {
                const int64_t gi = (qa + gq) * (P / 32) + pbase / 32;
                GroupCodes res;
                if constexpr (!DENSE) rotate_group(v[gq], c, sign_word);
                quantize_group_regs<MODE, false>(v[gq], seed_base ? seed + *seed_base : seed, gi, res);
                if (dequant) store_dequant<T>(reinterpret_cast<T*>(dequant) + gi * 32, res);
                ocodes[(lane * GPL + gq) * 4 + wave] = make_uint4(res.w[0], res.w[1], res.w[2], res.w[3]);
                reinterpret_cast<uint8_t*>(oscales)[(lane * GPL + gq) * 4 + wave] = (uint8_t)res.scale_byte;
            }
        }
        __syncthreads();
        const int64_t code_pitch = P / 2, scale_pitch = P / 32;
        for (int idx = tid; idx < TQ * 4; idx += 256) {
            const int ql = idx >> 2, part = idx & 3;
            if (q0 + ql < Q && p0 + part * 32 < P) {
                // tiled: this workgroup's 128 p are one 64-byte column block, so 16 consecutive q rows form one 1 KiB tile
                const int64_t off = tiled_out ? tiled_code_offset(q0 + ql, p0 / 128, P / 128) + part * 16
                                              : (q0 + ql) * code_pitch + p0 / 2 + part * 16;
                *reinterpret_cast<uint4*>(codes + off) = ocodes[idx];
            }
        }
        if (tid < TQ && q0 + tid < Q) {
            const uint32_t sw = oscales[tid];
            uint8_t* dst = scales + (q0 + tid) * scale_pitch + p0 / 32;
            if (p0 + kTrP <= P) {
                *reinterpret_cast<uint32_t*>(dst) = sw;
            } else {
                for (int b = 0; b < 4; ++b)
                    if (p0 + b * 32 < P) dst[b] = (uint8_t)(sw >> (8 * b));
            }
        }
    }
};

// ---- packed MXFP4 in, transposed + rotated + re-quantized out --------------------------------------------
// in: codes [R, C/2], scales [R, C/32]; out: the [C, R] tensor quantized along R.  A wave owns 128 rows by 64
// columns: lane l reads, for the 32 rows of row group l / 16, the two code bytes (four columns c) at byte column
// 2 (l % 16) straight from global memory -- a wave load is four contiguous 32-byte row segments, two rows share a
// register -- plus the rows' E8M0 byte of its column group.  It then handles its four columns two at a time: the
// hardware FP4 de-quantizing convert turns one byte of each row into two floats, which gives two groups of 32 along r
// in registers.  A workgroup stacks its four waves along r (512 rows), so that a column's scale bytes leave as one
// 16-byte piece; codes leave through LDS as whole 64-byte row pieces (tiled output: four contiguous 1 KiB tiles per wave).
constexpr int kRqR = 512, kRqC = 64;

template <int VAL_DTYPE, int MODE, bool DENSE = false>
struct RequantJob {
    const uint8_t* codes_in;
    const uint8_t* scales_in;
    int64_t R, C;
    float post, c;
    uint32_t sign_word;
    uint64_t seed;
    const uint64_t* seed_base = nullptr;  // device memory, or null: a value the kernel adds to `seed` when it runs
    uint8_t* codes;
    uint8_t* scales;
    void* dequant;
    bool tiled_in, tiled_out;
    const float* matrix;  // DENSE: the rotation, [32][32] fp32 (c and sign_word are then unused)
    unsigned grid_r, blocks;

    RequantJob(const uint8_t* codes_in_, const uint8_t* scales_in_, int64_t R_, int64_t C_, float post_, float c_,
               uint32_t sign_word_, uint64_t seed_, uint8_t* codes_, uint8_t* scales_, void* dequant_, bool tiled_in_,
               bool tiled_out_, const float* matrix_ = nullptr)
        : codes_in(codes_in_), scales_in(scales_in_), R(R_), C(C_), post(post_), c(c_), sign_word(sign_word_), seed(seed_),
          codes(codes_), scales(scales_), dequant(dequant_), tiled_in(tiled_in_), tiled_out(tiled_out_), matrix(matrix_),
          grid_r((unsigned)((R_ + kRqR - 1) / kRqR)),
          blocks((unsigned)(((R_ + kRqR - 1) / kRqR) * ((C_ + kRqC - 1) / kRqC))) {}

    // columns 2 P and 2 P + 1 of the lane's four: de-quantize byte P of the 32 rows, rotate, quantize, stage
    template <int P>
    __device__ __forceinline__ void column_pair(const uint32_t (&cw)[16], const float (&sc)[32], const DenseFrag& frag, bool active,
                                                int64_t ca, int64_t rbase, int cq, int rg, int wave, uint4* ocodes,
                                                uint8_t* oscales) const {
        using T = typename std::conditional<VAL_DTYPE == BF16, uint16_t, float>::type;
        float v[2][32];
#pragma unroll
        for (int i = 0; i < 32; i += 2) {
            // cw[i / 2]: bytes 0, 1 = row i, bytes 2, 3 = row i + 1
            const v2f pr0 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(cw[i >> 1], sc[i], P);
            const v2f pr1 = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(cw[i >> 1], sc[i + 1], 2 + P);
            v[0][i] = pr0.x; v[1][i] = pr0.y;
            v[0][i + 1] = pr1.x; v[1][i + 1] = pr1.y;
        }
        if (post != 1.0f) {  // absmax-coded input: value = code * 2^k * post, held in val_dtype
#pragma unroll
            for (int gq = 0; gq < 2; ++gq)
#pragma unroll
                for (int i = 0; i < 32; ++i) {
                    float a = v[gq][i] * post;
                    if constexpr (VAL_DTYPE == BF16) a = bf16_to_f32(f32_to_bf16(a));
                    v[gq][i] = a;
                }
        }
        if constexpr (DENSE) {  // the matrix instruction needs the whole wave, lanes outside the tensor included
            dense_rotate(v[0], frag);
            dense_rotate(v[1], frag);
        }
        if (!active) return;
#pragma unroll
        for (int gq = 0; gq < 2; ++gq) {
            const int64_t gi = (ca + 2 * P + gq) * (R / 32) + rbase / 32;
            GroupCodes res;
            if constexpr (!DENSE) rotate_group(v[gq], c, sign_word);
            quantize_group_regs<MODE, false>(v[gq], seed_base ? seed + *seed_base : seed, gi, res);
            if (dequant) store_dequant<T>(reinterpret_cast<T*>(dequant) + gi * 32, res);
            const int cl = 4 * cq + 2 * P + gq;
            ocodes[cl * 4 + rg] = make_uint4(res.w[0], res.w[1], res.w[2], res.w[3]);
            oscales[cl * 16 + wave * 4 + rg] = (uint8_t)res.scale_byte;
        }
    }

    __device__ __forceinline__ void run(unsigned bid) const {
        __shared__ uint4 ocodes_all[4][kRqC * 4];  // per wave: [c][4 row groups x 16 B]
        __shared__ uint4 oscales_all[kRqC];        // [c][16 scale bytes: wave-major, then row group]
        const int tid = threadIdx.x, lane = tid & 63;
        const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // tells the compiler it is wave-uniform
        const unsigned bc = bid / grid_r;
        const int64_t r0 = (int64_t)(bid - bc * grid_r) * kRqR, c0 = (int64_t)bc * kRqC;
        const int64_t in_code_pitch = C / 2, in_scale_pitch = C / 32;
        const int64_t rw = r0 + wave * 128;          // this wave's first row
        const int rg = lane >> 4, cq = lane & 15;    // row group within the wave, column quad
        const int64_t rbase = rw + 32 * rg;
        const int64_t ca = c0 + 4 * cq;              // this lane's first column
        const bool active = rbase < R && ca < C;     // R % 32 == 0 and C % 32 == 0: all of a lane's groups or none
        uint32_t cw[16];
        float sc[32];
        if (active) {
            // Uniform row pointers (scalar unit) + the lane's 32-bit byte offset: no per-lane 64-bit address math.
            // Tiled input: rows are 64 bytes apart inside a 16-row block, blocks (C / 128) KiB apart.
            const int64_t blk = (C / 128) * 1024;
            const uint8_t* cu = tiled_in ? codes_in + tiled_code_offset(rw, c0 / 128, C / 128) + (c0 & 127) / 2
                                         : codes_in + rw * in_code_pitch + c0 / 2;
            const uint32_t lane_off = (uint32_t)((tiled_in ? 2 * rg * blk : 32 * rg * in_code_pitch) + 2 * cq);
            const int64_t row_step = tiled_in ? 64 : in_code_pitch;                 // next row of a 16-row block
            const int64_t block_step = tiled_in ? blk - 16 * 64 : 0;                // extra hop into the next block
            const uint8_t* su = scales_in + rw * in_scale_pitch + c0 / 32;
            const uint32_t slane_off = (uint32_t)(32 * rg * in_scale_pitch + (cq >> 3));
#pragma unroll
            for (int i = 0; i < 32; i += 2) {
                const uint32_t lo = *reinterpret_cast<const uint16_t*>(cu + i * row_step + (i >> 4) * block_step + lane_off);
                const uint32_t hi = *reinterpret_cast<const uint16_t*>(cu + (i + 1) * row_step + (i >> 4) * block_step + lane_off);
                cw[i >> 1] = lo | (hi << 16);
            }
#pragma unroll
            for (int i = 0; i < 32; ++i) sc[i] = u2f((uint32_t)(su + i * in_scale_pitch)[slane_off] << 23);
        } else {
#pragma unroll
            for (int i = 0; i < 16; ++i) cw[i] = 0u;
#pragma unroll
            for (int i = 0; i < 32; ++i) sc[i] = 1.0f;
        }
        job_requests_issued();
        DenseFrag frag;
        if constexpr (DENSE) load_dense_frag(matrix, VAL_DTYPE, frag);
        uint4* ocodes = ocodes_all[wave];
        uint8_t* oscales = reinterpret_cast<uint8_t*>(oscales_all);
        column_pair<0>(cw, sc, frag, active, ca, rbase, cq, rg, wave, ocodes, oscales);
        column_pair<1>(cw, sc, frag, active, ca, rbase, cq, rg, wave, ocodes, oscales);
        __syncthreads();
        const int64_t code_pitch = R / 2, scale_pitch = R / 32;
        // codes: each wave writes its own 64 x 64-byte tile
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const int idx = it * 64 + lane, cl = idx >> 2, part = idx & 3;
            if (c0 + cl < C && rw + part * 32 < R) {
                const int64_t off = tiled_out ? tiled_code_offset(c0 + cl, rw / 128, R / 128) + part * 16
                                              : (c0 + cl) * code_pitch + rw / 2 + part * 16;
                *reinterpret_cast<uint4*>(codes + off) = ocodes[idx];
            }
        }
        // scales: one column's 16 bytes (the workgroup's 512 rows) per thread
        if (tid < kRqC && c0 + tid < C) {
            const uint4 sw = oscales_all[tid];
            uint8_t* dst = scales + (c0 + tid) * scale_pitch + r0 / 32;
            if (r0 + kRqR <= R && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
                *reinterpret_cast<uint4*>(dst) = sw;
            } else {
                const uint32_t w4[4] = {sw.x, sw.y, sw.z, sw.w};
                for (int b = 0; b < 16; ++b)
                    if (r0 + b * 32 < R) dst[b] = (uint8_t)(w4[b >> 2] >> (8 * (b & 3)));
            }
        }
    }
};

template <typename T, bool DENSE>
void launch_transposed_g32(int mode, const void* x, int64_t P, int64_t Q, float c, uint32_t sign_word, uint64_t seed,
                           uint8_t* codes, uint8_t* scales, void* dequant, bool tiled, const float* matrix, hipStream_t stream) {
    switch (mode) {
        case QUEST_RTN: launch_job(TransposedJob<T, QUEST_RTN, DENSE>(x, P, Q, c, sign_word, seed, codes, scales, dequant, tiled, matrix), stream); break;
        case ABSMAX_RTN: launch_job(TransposedJob<T, ABSMAX_RTN, DENSE>(x, P, Q, c, sign_word, seed, codes, scales, dequant, tiled, matrix), stream); break;
        case ABSMAX_SR: launch_job(TransposedJob<T, ABSMAX_SR, DENSE>(x, P, Q, c, sign_word, seed, codes, scales, dequant, tiled, matrix), stream); break;
        default: launch_job(TransposedJob<T, QUEST_SR, DENSE>(x, P, Q, c, sign_word, seed, codes, scales, dequant, tiled, matrix), stream); break;
    }
}

template <int VAL_DTYPE, bool DENSE>
void launch_requant_g32(int mode, const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C, float post,
                        float c, uint32_t sign_word, uint64_t seed, uint8_t* codes, uint8_t* scales, void* dequant,
                        bool tiled_in, bool tiled_out, const float* matrix, hipStream_t stream) {
    switch (mode) {
        case QUEST_RTN: launch_job(RequantJob<VAL_DTYPE, QUEST_RTN, DENSE>(codes_in, scales_in, R, C, post, c, sign_word, seed, codes, scales, dequant, tiled_in, tiled_out, matrix), stream); break;
        case ABSMAX_RTN: launch_job(RequantJob<VAL_DTYPE, ABSMAX_RTN, DENSE>(codes_in, scales_in, R, C, post, c, sign_word, seed, codes, scales, dequant, tiled_in, tiled_out, matrix), stream); break;
        case ABSMAX_SR: launch_job(RequantJob<VAL_DTYPE, ABSMAX_SR, DENSE>(codes_in, scales_in, R, C, post, c, sign_word, seed, codes, scales, dequant, tiled_in, tiled_out, matrix), stream); break;
        default: launch_job(RequantJob<VAL_DTYPE, QUEST_SR, DENSE>(codes_in, scales_in, R, C, post, c, sign_word, seed, codes, scales, dequant, tiled_in, tiled_out, matrix), stream); break;
    }
}

}  // namespace

// hd = 32, row-major input, RTN or Philox-driven SR (explicit uniforms take the generic path); rotate = false
// quantizes groups of 32 as they are (input rotated by the caller)
hipError_t quantize_rowmajor_hd32(const void* x, int dtype, int64_t rows, int64_t cols, uint32_t sign_word, int mode,
                                  uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                                  bool tiled, bool rotate, hipStream_t stream) {
    if (!rotate && (tiled || sign_word)) return hipErrorInvalidValue;  // pass-through groups: row-major codes, no signs
    GroupOut out{reinterpret_cast<uint4*>(codes), scales, reinterpret_cast<uint32_t*>(maskbits), dequant};
    const float c = rotate ? hadamard_scale(32, dtype) : 1.0f;
    if (maskbits) {
        if (dtype == BF16) launch_rowmajor_g32<uint16_t, true>(mode, x, rows, cols, tiled, c, sign_word, seed, out, rotate, stream);
        else launch_rowmajor_g32<float, true>(mode, x, rows, cols, tiled, c, sign_word, seed, out, rotate, stream);
    } else {
        if (dtype == BF16) launch_rowmajor_g32<uint16_t, false>(mode, x, rows, cols, tiled, c, sign_word, seed, out, rotate, stream);
        else launch_rowmajor_g32<float, false>(mode, x, rows, cols, tiled, c, sign_word, seed, out, rotate, stream);
    }
    return hipGetLastError();
}

// hd = 64 or 128, row-major input, RTN or Philox-driven SR, row-major codes
hipError_t quantize_rowmajor_wide(const void* x, int dtype, int64_t n, int hd, const SignBits& sb, int mode, uint64_t seed,
                                  uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant, hipStream_t stream) {
    GroupOut out{reinterpret_cast<uint4*>(codes), scales, reinterpret_cast<uint32_t*>(maskbits), dequant};
    const float c = hadamard_scale(hd, dtype);
    const auto go = [&](auto tag, auto mask, auto hdc) {
        using T = decltype(tag);
        launch_rowmajor_wide<T, decltype(mask)::value, decltype(hdc)::value>(mode, x, n, c, sb, seed, out, stream);
    };
    const auto by_hd = [&](auto tag, auto mask) {
        if (hd == 64) go(tag, mask, std::integral_constant<int, 64>{});
        else go(tag, mask, std::integral_constant<int, 128>{});
    };
    if (maskbits) {
        if (dtype == BF16) by_hd(uint16_t{}, std::true_type{});
        else by_hd(float{}, std::true_type{});
    } else {
        if (dtype == BF16) by_hd(uint16_t{}, std::false_type{});
        else by_hd(float{}, std::false_type{});
    }
    return hipGetLastError();
}

// hd = 32, x is [P, Q] row-major and the output is its transpose quantized along P; no clip mask
hipError_t quantize_transposed_hd32(const void* x, int dtype, int64_t P, int64_t Q, uint32_t sign_word, int mode,
                                    uint64_t seed, uint8_t* codes, uint8_t* scales, void* dequant, bool tiled,
                                    hipStream_t stream) {
    const float c = hadamard_scale(32, dtype);
    if (dtype == BF16) launch_transposed_g32<uint16_t, false>(mode, x, P, Q, c, sign_word, seed, codes, scales, dequant, tiled, nullptr, stream);
    else launch_transposed_g32<float, false>(mode, x, P, Q, c, sign_word, seed, codes, scales, dequant, tiled, nullptr, stream);
    return hipGetLastError();
}

hipError_t requantize_transposed_hd32(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C, float post,
                                      int val_dtype, uint32_t sign_word, int mode, uint64_t seed, uint8_t* codes,
                                      uint8_t* scales, void* dequant, bool tiled_in, bool tiled_out, hipStream_t stream) {
    const float c = hadamard_scale(32, val_dtype);
    if (val_dtype == BF16) launch_requant_g32<BF16, false>(mode, codes_in, scales_in, R, C, post, c, sign_word, seed, codes, scales, dequant, tiled_in, tiled_out, nullptr, stream);
    else launch_requant_g32<F32, false>(mode, codes_in, scales_in, R, C, post, c, sign_word, seed, codes, scales, dequant, tiled_in, tiled_out, nullptr, stream);
    return hipGetLastError();
}

// ---- the same three with a dense 32x32 rotation (matrix: device pointer to [32][32] fp32, H[k][j]; its entries are
// rounded to the tensor's dtype as the reference casts its matrix, quantizers/mxfp4.py:49) ---------------------------
hipError_t quantize_rowmajor_dense(const void* x, int dtype, int64_t rows, int64_t cols, const float* matrix, int mode,
                                   uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                                   bool tiled, hipStream_t stream) {
    GroupOut out{reinterpret_cast<uint4*>(codes), scales, reinterpret_cast<uint32_t*>(maskbits), dequant};
    if (maskbits) {
        if (dtype == BF16) launch_rowmajor_dense<uint16_t, true>(mode, x, rows, cols, matrix, seed, out, tiled, stream);
        else launch_rowmajor_dense<float, true>(mode, x, rows, cols, matrix, seed, out, tiled, stream);
    } else {
        if (dtype == BF16) launch_rowmajor_dense<uint16_t, false>(mode, x, rows, cols, matrix, seed, out, tiled, stream);
        else launch_rowmajor_dense<float, false>(mode, x, rows, cols, matrix, seed, out, tiled, stream);
    }
    return hipGetLastError();
}

hipError_t quantize_transposed_dense(const void* x, int dtype, int64_t P, int64_t Q, const float* matrix, int mode,
                                     uint64_t seed, uint8_t* codes, uint8_t* scales, void* dequant, bool tiled,
                                     hipStream_t stream) {
    if (dtype == BF16) launch_transposed_g32<uint16_t, true>(mode, x, P, Q, 1.0f, 0u, seed, codes, scales, dequant, tiled, matrix, stream);
    else launch_transposed_g32<float, true>(mode, x, P, Q, 1.0f, 0u, seed, codes, scales, dequant, tiled, matrix, stream);
    return hipGetLastError();
}

hipError_t requantize_transposed_dense(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C, float post,
                                       int val_dtype, const float* matrix, int mode, uint64_t seed, uint8_t* codes,
                                       uint8_t* scales, void* dequant, bool tiled_in, bool tiled_out, hipStream_t stream) {
    if (val_dtype == BF16) launch_requant_g32<BF16, true>(mode, codes_in, scales_in, R, C, post, 1.0f, 0u, seed, codes, scales, dequant, tiled_in, tiled_out, matrix, stream);
    else launch_requant_g32<F32, true>(mode, codes_in, scales_in, R, C, post, 1.0f, 0u, seed, codes, scales, dequant, tiled_in, tiled_out, matrix, stream);
    return hipGetLastError();
}

// ---- producers fused into the forward quantizer ------------------------------------------------------------------
// The tensor the model would hand to the quantized linear (RMSNorm output, src/models/llama.py:64-75; SwiGLU product,
// llama.py:113-114) is computed group by group in registers and never written.  One wave owns one row: lane l takes
// groups l, l+64, ... of 32 consecutive elements, so a row of up to 2048 elements is read exactly once.

namespace {

typedef __bf16 v2bf16 __attribute__((ext_vector_type(2)));
// round to bf16 and back (round to nearest even, v_cvt_pk_bf16_f32)
__device__ __forceinline__ void round_pair_to_bf16(float& a, float& b) {
    const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{a, b}, v2bf16));
    a = u2f(w << 16);
    b = u2f(w & 0xffff0000u);
}

// TA = void: plain.  Otherwise the norm's input is x + add (the residual sum in front of the norm, src/models/llama.py:
// 170-171), formed here in T's arithmetic and written to xsum, which the rest of the model continues with.
template <typename T, typename TA = void>
struct RmsNormProducer {
    static constexpr int kOutDtype = F32;  // bf16-or-fp32 normalised value times the fp32 gain is fp32
    static constexpr bool kAdd = !std::is_void<TA>::value;
    using TAdd = typename std::conditional<kAdd, TA, T>::type;
    const T* x;
    const float* gain;
    float* factor;  // [rows]: 1 / sqrt(mean(x^2) + eps), kept for the backward pass
    float eps;
    const TAdd* add;
    T* xsum;

    // 8 KiB of LDS per wave of the workgroup: staging of the residual sum on its way out
    __device__ __forceinline__ static float4* xsum_area() {
        __shared__ float4 xbuf[4][512];
        return xbuf[threadIdx.x >> 6];
    }

    // The row's factor; `first` leaves with the raw elements of the lane's first group (if it has one).
    // Sum of squares in a fixed order: sixteen interleaved partial sums (partial j adds the sums of groups j, j+16,
    // j+32, ... in ascending order, each group summed by the pairwise tree), then the pairwise tree over the sixteen.
    // A lane without a group adds +0, which leaves a sum of squares unchanged.
    // W < 64: the wave holds 64 / W rows of at most W groups each, a row in the W lanes from `seg` on (`lane` counts
    // from there); the partial sums then have W / 16 terms instead of four, the missing ones being the +0 of above.
    template <int W = 64>
    __device__ __forceinline__ float prepare(int64_t row, int lane, int groups, int64_t cols, float (&first)[32], int seg = 0) const {
        float acc = 0.0f;
        for (int base = 0; base < groups; base += 64) {
            const int g = base + lane;
            float s = 0.0f;
            if (g < groups) {
                float v[32];
                load_group<T>(x + row * cols + g * 32, v);
                if constexpr (kAdd) {
                    static_assert(!kAdd || sizeof(T) == 4, "the residual sum is formed in fp32");
                    float a[32];
                    load_group<TAdd>(add + row * cols + g * 32, a);
#pragma unroll
                    for (int i = 0; i < 32; ++i) v[i] = v[i] + a[i];
                    if constexpr (W == 64) {
                        // the sum leaves through LDS so that an instruction stores whole 128-byte lines (a lane's own
                        // 128 bytes would go out as eight 16-byte pieces of 64 different lines per instruction); slot
                        // 8 l + (q ^ l % 8) of the wave's area holds piece q of lane l's group: writes and the
                        // slot-ordered reads both spread over all banks
                        float4* area = xsum_area();
#pragma unroll
                        for (int q = 0; q < 8; ++q)
                            area[8 * lane + (q ^ (lane & 7))] = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
                    } else {
                        float4* dst = reinterpret_cast<float4*>(xsum + row * cols + g * 32);
#pragma unroll
                        for (int q = 0; q < 8; ++q) dst[q] = make_float4(v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]);
                    }
                }
                if (base == 0) {
#pragma unroll
                    for (int i = 0; i < 32; ++i) first[i] = v[i];
                }
#pragma unroll
                for (int i = 0; i < 32; ++i) v[i] = v[i] * v[i];
                s = tree_sum32(v);
            }
            if constexpr (kAdd && W == 64) {
                const float4* area = xsum_area();
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    const int slot = 64 * i + lane, gl = slot >> 3, piece = (slot & 7) ^ (gl & 7);
                    if (base + gl < groups)
                        reinterpret_cast<float4*>(xsum + row * cols + (int64_t)(base + gl) * 32)[piece] = area[slot];
                }
                __builtin_amdgcn_wave_barrier();  // the next pass over the row reuses the area
            }
#pragma unroll
            for (int k = 0; k < W / 16; ++k) acc = acc + __shfl(s, seg + (lane & 15) + 16 * k, 64);
        }
#pragma unroll
        for (int m = 1; m < 16; m <<= 1) acc = acc + __shfl_xor(acc, m, 64);
        const float f = 1.0f / __builtin_sqrtf(acc / (float)cols + eps);
        if (lane == 0) factor[row] = f;
        return f;
    }
    // v holds the group's raw elements on entry when have_raw
    __device__ __forceinline__ void load(int64_t row, int g, int64_t cols, float f, bool have_raw, float (&v)[32]) const {
        // with a residual sum: the lane reads back what it stored in prepare()
        if (!have_raw) load_group<T>((kAdd ? xsum : x) + row * cols + g * 32, v);
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = v[i] * f;
        if constexpr (sizeof(T) == 2) {  // .type_as(x)
#pragma unroll
            for (int i = 0; i < 32; i += 2) round_pair_to_bf16(v[i], v[i + 1]);
        }
        float w[32];
        load_group<float>(gain + g * 32, w);
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = v[i] * w[i];
    }
};

template <typename T>
struct SwiGluProducer {
    static constexpr int kOutDtype = sizeof(T) == 2 ? BF16 : F32;
    const T* h12;  // [rows, 2 cols]: up, then gate

    template <int W = 64>
    __device__ __forceinline__ float prepare(int64_t, int, int, int64_t, float (&)[32], int = 0) const { return 0.0f; }
    __device__ __forceinline__ void load(int64_t row, int g, int64_t cols, float, bool, float (&v)[32]) const {
        float gate[32];
        load_group<T>(h12 + row * 2 * cols + g * 32, v);
        load_group<T>(h12 + row * 2 * cols + cols + g * 32, gate);
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = silu_fixed(v[i]);
        if constexpr (sizeof(T) == 2) {  // a bf16 tensor rounds after each op
#pragma unroll
            for (int i = 0; i < 32; i += 2) round_pair_to_bf16(v[i], v[i + 1]);
        }
#pragma unroll
        for (int i = 0; i < 32; ++i) v[i] = v[i] * gate[i];
        if constexpr (sizeof(T) == 2) {
#pragma unroll
            for (int i = 0; i < 32; i += 2) round_pair_to_bf16(v[i], v[i + 1]);
        }
    }
};

// quest RTN + clip mask (the forward quantizer) of rows that a producer computes
// W: lanes per row (64, or 32 / 16 for rows of at most that many groups: two / four rows per wave)
template <typename P, bool TILED, int W = 64>
struct ProducedRowsJob {
    P prod;
    int64_t rows, cols;
    float c;
    uint32_t sign_word;
    GroupOut out;
    unsigned blocks;

    ProducedRowsJob(const P& prod_, int64_t rows_, int64_t cols_, uint32_t sign_word_, const GroupOut& out_)
        : prod(prod_), rows(rows_), cols(cols_), c(hadamard_scale(32, P::kOutDtype)), sign_word(sign_word_), out(out_),
          blocks((unsigned)((rows_ + 4 * (64 / W) - 1) / (4 * (64 / W)))) {}

    __device__ __forceinline__ void run(unsigned bid) const {
        const int wlane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const int lane = wlane & (W - 1), seg = wlane - lane;  // place in the row's segment of the wave
        int64_t row = ((int64_t)bid * 4 + wave) * (64 / W) + seg / W;
        if (row - seg / W >= rows) return;  // a whole wave
        if (row >= rows) row = rows - 1;    // a segment past the end repeats the last row: same values to the same places
        const int groups = (int)(cols / 32);
        float v[32];
        const float state = prod.template prepare<W>(row, lane, groups, cols, v, seg);
        // TILED: cols % 128 == 0, so the four lanes of a quad run the same number of iterations
        for (int g = lane; g < groups; g += W) {
            const int64_t gi = row * groups + g;
            const int64_t ci = TILED ? (row >> 4) * 16 * groups + ((g >> 2) * 64 + (int)(row & 15) * 4 + (g & 3)) : gi;
            prod.load(row, g, cols, state, g == lane, v);
            rotate_group(v, c, sign_word);
            GroupCodes o;
            quantize_group_regs<QUEST_RTN, true>(v, 0, gi, o);
            out.codes[ci] = make_uint4(o.w[0], o.w[1], o.w[2], o.w[3]);
            if constexpr (TILED) {
                const uint32_t s1 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)o.scale_byte, 0x55, 0xf, 0xf, false);
                const uint32_t s2 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)o.scale_byte, 0xAA, 0xf, 0xf, false);
                const uint32_t s3 = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)o.scale_byte, 0xFF, 0xf, 0xf, false);
                if ((lane & 3) == 0)
                    *reinterpret_cast<uint32_t*>(out.scales + gi) = o.scale_byte | (s1 << 8) | (s2 << 16) | (s3 << 24);
            } else {
                out.scales[gi] = (uint8_t)o.scale_byte;
            }
            out.maskbits[gi] = o.keep;
        }
    }
};

template <typename P, int W>
void launch_produced_w(const P& prod, int64_t rows, int64_t cols, uint32_t sign_word, const GroupOut& out, bool tiled,
                       hipStream_t stream) {
    if (tiled) launch_job(ProducedRowsJob<P, true, W>(prod, rows, cols, sign_word, out), stream);
    else launch_job(ProducedRowsJob<P, false, W>(prod, rows, cols, sign_word, out), stream);
}

template <typename P>
void launch_produced(const P& prod, int64_t rows, int64_t cols, uint32_t sign_word, uint8_t* codes, uint8_t* scales,
                     uint8_t* maskbits, bool tiled, hipStream_t stream) {
    const GroupOut out{reinterpret_cast<uint4*>(codes), scales, reinterpret_cast<uint32_t*>(maskbits), nullptr};
    if (cols <= 16 * 32) launch_produced_w<P, 16>(prod, rows, cols, sign_word, out, tiled, stream);
    else if (cols <= 32 * 32) launch_produced_w<P, 32>(prod, rows, cols, sign_word, out, tiled, stream);
    else launch_produced_w<P, 64>(prod, rows, cols, sign_word, out, tiled, stream);
}

}  // namespace

// Q(rmsnorm(x) * gain): Hadamard block 32, quest RTN, clip mask; factor [rows] receives 1 / sqrt(mean(x^2) + eps).
// add != null (x fp32 only): the norm's input is x + add, also written to xsum [rows, cols] fp32.
hipError_t rmsnorm_quantize_hd32(const void* x, int dtype, const void* add, int add_dtype, void* xsum, const float* gain, float eps,
                                 int64_t rows, int64_t cols, uint32_t sign_word, uint8_t* codes, uint8_t* scales, uint8_t* maskbits,
                                 float* factor, bool tiled, hipStream_t stream) {
    if (rows == 0) return hipSuccess;
    if (add) {
        if (dtype != F32) return hipErrorInvalidValue;
        const float* xp = reinterpret_cast<const float*>(x);
        float* sp = reinterpret_cast<float*>(xsum);
        if (add_dtype == BF16)
            launch_produced(RmsNormProducer<float, uint16_t>{xp, gain, factor, eps, reinterpret_cast<const uint16_t*>(add), sp}, rows,
                            cols, sign_word, codes, scales, maskbits, tiled, stream);
        else
            launch_produced(RmsNormProducer<float, float>{xp, gain, factor, eps, reinterpret_cast<const float*>(add), sp}, rows, cols,
                            sign_word, codes, scales, maskbits, tiled, stream);
    } else if (dtype == BF16) {
        launch_produced(RmsNormProducer<uint16_t>{reinterpret_cast<const uint16_t*>(x), gain, factor, eps, nullptr, nullptr}, rows,
                        cols, sign_word, codes, scales, maskbits, tiled, stream);
    } else {
        launch_produced(RmsNormProducer<float>{reinterpret_cast<const float*>(x), gain, factor, eps, nullptr, nullptr}, rows, cols,
                        sign_word, codes, scales, maskbits, tiled, stream);
    }
    return hipGetLastError();
}

// Q(silu(up) * gate) of h12 [rows, 2 hidden] = (up, gate): Hadamard block 32, quest RTN, clip mask
hipError_t swiglu_quantize_hd32(const void* h12, int dtype, int64_t rows, int64_t hidden, uint32_t sign_word,
                                uint8_t* codes, uint8_t* scales, uint8_t* maskbits, bool tiled, hipStream_t stream) {
    if (rows == 0) return hipSuccess;
    if (dtype == BF16)
        launch_produced(SwiGluProducer<uint16_t>{reinterpret_cast<const uint16_t*>(h12)}, rows, hidden, sign_word, codes,
                        scales, maskbits, tiled, stream);
    else
        launch_produced(SwiGluProducer<float>{reinterpret_cast<const float*>(h12)}, rows, hidden, sign_word, codes, scales,
                        maskbits, tiled, stream);
    return hipGetLastError();
}

// ---- two independent jobs per launch (the whole-layer entry points) ---------------------------------------------

namespace {
template <typename F>
void with_elem_type(int dtype, F&& f) {
    if (dtype == BF16) f(uint16_t{});
    else f(float{});
}
template <typename F>
void with_absmax_mode(int mode, F&& f) {
    if (mode == ABSMAX_SR) f(std::integral_constant<int, ABSMAX_SR>{});
    else f(std::integral_constant<int, ABSMAX_RTN>{});
}
}  // namespace

// forward quantizer (quest RTN + clip mask, tiled codes) of two tensors, e.g. the activations and the weight of a layer
hipError_t quantize_rowmajor_hd32_tiled_pair(const RowmajorArgs& a, const RowmajorArgs& b, hipStream_t stream) {
    const GroupOut oa{reinterpret_cast<uint4*>(a.codes), a.scales, reinterpret_cast<uint32_t*>(a.maskbits), nullptr};
    const GroupOut ob{reinterpret_cast<uint4*>(b.codes), b.scales, reinterpret_cast<uint32_t*>(b.maskbits), nullptr};
    const float ca = hadamard_scale(32, a.dtype), cb = hadamard_scale(32, b.dtype);
    with_elem_type(a.dtype, [&](auto ta) {
        with_elem_type(b.dtype, [&](auto tb) {
            launch_job_pair(RowmajorTiledJob<decltype(ta), QUEST_RTN, true>(a.x, a.rows, a.cols, ca, a.sign_word, 0, oa),
                            RowmajorTiledJob<decltype(tb), QUEST_RTN, true>(b.x, b.rows, b.cols, cb, b.sign_word, 0, ob), stream);
        });
    });
    return hipGetLastError();
}

// absmax quantizer of e [T, O] along its rows and of its transpose along T, tiled codes, one pass of launches
hipError_t quantize_both_orientations_hd32_tiled(const void* e, int dtype, int64_t T, int64_t O, uint32_t sign_word, int mode,
                                                 uint64_t seed_rows, uint64_t seed_transposed, uint8_t* codes_rows,
                                                 uint8_t* scales_rows, uint8_t* codes_transposed, uint8_t* scales_transposed,
                                                 const uint64_t* seed_base, hipStream_t stream) {
    const GroupOut orow{reinterpret_cast<uint4*>(codes_rows), scales_rows, nullptr, nullptr};
    const float c = hadamard_scale(32, dtype);
    with_elem_type(dtype, [&](auto t) {
        with_absmax_mode(mode, [&](auto m) {
            using T_ = decltype(t);
            constexpr int M = decltype(m)::value;
            TransposedJob<T_, M> jt(e, T, O, c, sign_word, seed_transposed, codes_transposed, scales_transposed, nullptr, true);
            RowmajorTiledJob<T_, M, false> jr(e, T, O, c, sign_word, seed_rows, orow);
            jt.seed_base = jr.seed_base = seed_base;
            launch_job_pair(jt, jr, stream);
        });
    });
    return hipGetLastError();
}

// transpose + rotate + re-quantize two packed tensors (tiled codes in and out), e.g. Q(W) and Q(x) of a layer
hipError_t requantize_transposed_hd32_tiled_pair(const RequantArgs& a, const RequantArgs& b, uint32_t sign_word, int mode,
                                                 const uint64_t* seed_base, hipStream_t stream) {
    const float ca = hadamard_scale(32, a.val_dtype), cb = hadamard_scale(32, b.val_dtype);
    const auto with_val = [](int dt, auto&& f) {
        if (dt == BF16) f(std::integral_constant<int, BF16>{});
        else f(std::integral_constant<int, F32>{});
    };
    with_val(a.val_dtype, [&](auto va) {
        with_val(b.val_dtype, [&](auto vb) {
            with_absmax_mode(mode, [&](auto m) {
                constexpr int M = decltype(m)::value;
                RequantJob<decltype(va)::value, M> ja(a.codes_in, a.scales_in, a.R, a.C, 1.0f, ca, sign_word, a.seed, a.codes, a.scales, nullptr, true, true);
                RequantJob<decltype(vb)::value, M> jb(b.codes_in, b.scales_in, b.R, b.C, 1.0f, cb, sign_word, b.seed, b.codes, b.scales, nullptr, true, true);
                ja.seed_base = jb.seed_base = seed_base;
                launch_job_pair(ja, jb, stream);
            });
        });
    });
    return hipGetLastError();
}

}  // namespace qm
