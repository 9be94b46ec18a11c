// Fused block-Hadamard rotation + MXFP4 quantizer for gfx950.
//
// Replaces the reference's Triton kernel src/models/quantization/quantizers/mxfp4_triton.py:19-174
// and, for the transposed / re-quantizing variants, the .T.contiguous() copies followed by that
// kernel in src/models/quantization/backward.py:73,81-82.
//
// Work decomposition ("octet" layout): every lane owns 8 consecutive elements along the
// quantization axis, so one MX group of 32 is 4 adjacent lanes and one Hadamard chunk of
// hd = 32/64/128 is 4/8/16 adjacent lanes.  Butterfly strides 1,2,4 run in registers, strides
// 8 and 16 through DPP quad permutes, strides 32 and 64 through lane shuffles.  The summation
// order (ascending strides; group sums as a pairwise tree) is the canonical one the parity tests
// pin, so FP4 codes and E8M0 scales are reproducible bit for bit.
//
// HBM traffic per element (bf16 in): 2 B read + 0.5 B codes + 1/32 B scale (+ 1/8 B mask bits).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "qm_kernels.h"
#include "qm_math.h"

namespace qm {

namespace {

__device__ __forceinline__ float dpp_quad_xor1(float v) {
    return u2f((uint32_t)__builtin_amdgcn_mov_dpp((int)f2u(v), 0xB1, 0xF, 0xF, true));
}
__device__ __forceinline__ float dpp_quad_xor2(float v) {
    return u2f((uint32_t)__builtin_amdgcn_mov_dpp((int)f2u(v), 0x4E, 0xF, 0xF, true));
}
template <int LANE_MASK>
__device__ __forceinline__ float lane_xor(float v) {
    if constexpr (LANE_MASK == 1) return dpp_quad_xor1(v);
    else if constexpr (LANE_MASK == 2) return dpp_quad_xor2(v);
    else return __shfl_xor(v, LANE_MASK, 64);
}

template <int LANE_MASK>
__device__ __forceinline__ void cross_lane_stage(float (&v)[8], int lane_in_chunk) {
    const bool upper = (lane_in_chunk & LANE_MASK) != 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float p = lane_xor<LANE_MASK>(v[i]);
        v[i] = upper ? (p - v[i]) : (v[i] + p);
    }
}

// v: 8 consecutive inputs of this lane.  Out: rotated values (x @ H with H = c * S * diag(signs)).
template <int HD>
__device__ __forceinline__ void rotate_octet(float (&v)[8], int lane_in_chunk, float c, uint32_t sign8) {
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (i & h) continue;
            float a = v[i], b = v[i + h];
            v[i] = a + b;
            v[i + h] = a - b;
        }
    }
    cross_lane_stage<1>(v, lane_in_chunk);
    cross_lane_stage<2>(v, lane_in_chunk);
    if constexpr (HD >= 64) cross_lane_stage<4>(v, lane_in_chunk);
    if constexpr (HD >= 128) cross_lane_stage<8>(v, lane_in_chunk);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float r = v[i] * c;
        v[i] = ((sign8 >> i) & 1u) ? -r : r;
    }
}

__device__ __forceinline__ float group_tree_sum(const float (&p)[8]) {
    float a = (p[0] + p[1]) + (p[2] + p[3]);
    float b = (p[4] + p[5]) + (p[6] + p[7]);
    float w = a + b;
    w = w + dpp_quad_xor1(w);
    w = w + dpp_quad_xor2(w);
    return w;
}

struct OctetResult {
    uint32_t codes;       // 8 nibbles, element i in bits [4i, 4i+4)
    uint32_t scale_byte;  // E8M0, identical in the 4 lanes of a group
    uint32_t keep_bits;   // bit i = |t_i| < 6
    float deq[8];
};

// g: rotated values of this lane (one quarter of an MX group).  u: uniforms (SR modes only).
template <int MODE>
__device__ __forceinline__ void quantize_octet(const float (&g)[8], const float (&u)[8], OctetResult& out) {
    constexpr bool kQuest = (MODE == QUEST_RTN || MODE == QUEST_SR);
    constexpr bool kSR = (MODE == ABSMAX_SR || MODE == QUEST_SR);
    float t[8];
    float scale;
    if constexpr (kQuest) {
        float sq[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) sq[i] = g[i] * g[i];
        float ms = group_tree_sum(sq) * 0.03125f;
        float m = group_tree_sum(g) * 0.03125f;
        float mm = m * m;
        float var = ms - mm;
        var = var > 0.0f ? var : 0.0f;
        float sd = __builtin_sqrtf(var);  // correctly rounded (hipcc default for fp32 sqrt)
        float gs = kQuestG * sd;
        float s = gs + 1e-8f;
        int E = (int)((f2u(s) >> 23) & 0xffu) - 127;
        E = E > 127 ? 127 : E;
        out.scale_byte = (uint32_t)(E + 127);
        scale = pow2i(E);
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] = scale_pow2(g[i], -E);
    } else {
        float a = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) a = fmaxf(a, fabsf(g[i]));
        a = fmaxf(a, dpp_quad_xor1(a));
        a = fmaxf(a, dpp_quad_xor2(a));
        if (a == 0.0f) {
            // log2(0) = -inf in the reference: every compare is false, output is -0
            out.codes = 0x88888888u;
            out.scale_byte = 0u;
            out.keep_bits = 0u;
#pragma unroll
            for (int i = 0; i < 8; ++i) out.deq[i] = -0.0f;
            return;
        }
        int k = (int)((f2u(a) >> 23) & 0xffu) - 129;
        k = k < -127 ? -127 : (k > 127 ? 127 : k);
        out.scale_byte = (uint32_t)(k + 127);
        scale = scale_pow2(kFourThirds, k);
#pragma unroll
        for (int i = 0; i < 8; ++i) t[i] = div_four_thirds(scale_pow2(g[i], -k));
    }
    uint32_t codes = 0u, keep = 0u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        float A = fabsf(t[i]);
        uint32_t neg = !(g[i] > 0.0f);  // sign of t, taken from g so that it survives underflow
        int mag;
        if constexpr (kSR) mag = sr_code(A, u[i]);
        else mag = rtn_code(A);
        codes |= ((uint32_t)mag | (neg << 3)) << (4 * i);
        keep |= (uint32_t)(A < 6.0f) << i;
        float q = e2m1_value(mag);
        out.deq[i] = (neg ? -q : q) * scale;
    }
    out.codes = codes;
    out.keep_bits = keep;
}

template <typename T>
struct Elem;
template <>
struct Elem<uint16_t> {
    static __device__ __forceinline__ float load(uint16_t h) { return bf16_to_f32(h); }
    static __device__ __forceinline__ uint16_t store(float f) { return f32_to_bf16(f); }
};
template <>
struct Elem<float> {
    static __device__ __forceinline__ float load(float f) { return f; }
    static __device__ __forceinline__ float store(float f) { return f; }
};

template <typename T>
__device__ __forceinline__ void load_octet(const T* p, float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        uint4 raw = *reinterpret_cast<const uint4*>(p);
        uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = u2f(w[i] << 16);
            v[2 * i + 1] = u2f(w[i] & 0xffff0000u);
        }
    } else {
        float4 a = *reinterpret_cast<const float4*>(p);
        float4 b = *reinterpret_cast<const float4*>(p + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
}

template <typename T>
__device__ __forceinline__ void store_octet(T* p, const float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
            w[i] = (uint32_t)f32_to_bf16(v[2 * i]) | ((uint32_t)f32_to_bf16(v[2 * i + 1]) << 16);
        *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

struct QuantOut {
    uint32_t* codes;    // [n/8] dwords
    uint8_t* scales;    // [n/32]
    uint8_t* maskbits;  // [n/8] or null
    void* dequant;      // [n] of T or null
};

// Everything after the 8 raw values of a lane are in registers; `octet` = flat offset / 8 in the
// logical (row-major, quantization axis last) output tensor.
template <typename T, int HD, int MODE>
__device__ __forceinline__ void process_octet(float (&v)[8], int lane_in_chunk, int64_t octet, float c,
                                              const SignBits& sb, const float* __restrict__ u, uint64_t seed,
                                              const QuantOut& out) {
    constexpr bool kSR = (MODE == ABSMAX_SR || MODE == QUEST_SR);
    const int j0 = lane_in_chunk * 8;
    const uint32_t sign8 = (sb.w[j0 >> 5] >> (j0 & 31)) & 0xffu;
    rotate_octet<HD>(v, lane_in_chunk, c, sign8);
    float uu[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if constexpr (kSR) {
        if (u != nullptr) {
            load_octet<float>(u + octet * 8, uu);
        } else {
            // sixteen elements share one Philox call: the two octets of a pair compute it twice
            Philox4 ph = philox_for_hexadecad(seed, (uint64_t)(octet >> 1));
#pragma unroll
            for (int i = 0; i < 8; ++i) uu[i] = uniform_from_field22(philox_field22(ph, (int)(octet & 1) * 8 + i));
        }
    }
    OctetResult r;
    quantize_octet<MODE>(v, uu, r);
    out.codes[octet] = r.codes;
    if ((octet & 3) == 0) out.scales[octet >> 2] = (uint8_t)r.scale_byte;
    if (out.maskbits) out.maskbits[octet] = (uint8_t)r.keep_bits;
    if (out.dequant) store_octet<T>(reinterpret_cast<T*>(out.dequant) + octet * 8, r.deq);
}

// ---- row-major input: quantization axis is the contiguous one -----------------------------
template <typename T, int HD, int MODE>
__global__ __launch_bounds__(256) void quantize_rowmajor_kernel(const T* __restrict__ x, int64_t n_octets, float c,
                                                                SignBits sb, const float* __restrict__ u,
                                                                uint64_t seed, QuantOut out) {
    const int64_t octet = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (octet >= n_octets) return;  // n is a multiple of HD, so a chunk is all-in or all-out
    float v[8];
    load_octet<T>(x + octet * 8, v);
    process_octet<T, HD, MODE>(v, (int)(octet & (HD / 8 - 1)), octet, c, sb, u, seed, out);
}

// ---- transposed input: x is [P, Q] row-major, output is the [Q, P] tensor quantized along P -----
constexpr int kTileP = 128;  // along the quantization axis (multiple of every hd)
constexpr int kTileQ = 64;

template <typename T, int HD, int MODE>
__global__ __launch_bounds__(256) void quantize_transposed_kernel(const T* __restrict__ x, int64_t P, int64_t Q,
                                                                  float c, SignBits sb, const float* __restrict__ u,
                                                                  uint64_t seed, QuantOut out) {
    // one extra dword per row keeps the column reads (stride = one row) off a single LDS bank
    constexpr int kPitch = kTileQ * (int)sizeof(T) / 4 + 1;  // dwords
    __shared__ uint32_t tile[kTileP * kPitch];
    const int64_t p0 = (int64_t)blockIdx.x * kTileP;
    const int64_t q0 = (int64_t)blockIdx.y * kTileQ;
    constexpr int kVec = 16 / (int)sizeof(T);       // elements per 16-byte load
    constexpr int kVecPerRow = kTileQ / kVec;
    for (int idx = threadIdx.x; idx < kTileP * kVecPerRow; idx += 256) {
        const int row = idx / kVecPerRow, cv = idx % kVecPerRow;
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (p0 + row < P && q0 + cv * kVec < Q)
            raw = *reinterpret_cast<const uint4*>(x + (p0 + row) * Q + q0 + cv * kVec);
        uint32_t* dst = tile + row * kPitch + cv * 4;
        dst[0] = raw.x; dst[1] = raw.y; dst[2] = raw.z; dst[3] = raw.w;
    }
    __syncthreads();
    constexpr int kOctPerQ = kTileP / 8;  // 16 lanes cover one q
    for (int oc = threadIdx.x; oc < kTileQ * kOctPerQ; oc += 256) {
        const int ql = oc / kOctPerQ, po = oc % kOctPerQ;
        if (p0 + po * 8 >= P || q0 + ql >= Q) continue;
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t* rowp = tile + (po * 8 + i) * kPitch;
            if constexpr (sizeof(T) == 2) {
                uint32_t w = rowp[ql >> 1];
                v[i] = (ql & 1) ? u2f(w & 0xffff0000u) : u2f(w << 16);
            } else {
                v[i] = u2f(rowp[ql]);
            }
        }
        const int64_t octet = ((q0 + ql) * P + p0) / 8 + po;
        process_octet<T, HD, MODE>(v, po & (HD / 8 - 1), octet, c, sb, u, seed, out);
    }
}

// ---- packed MXFP4 in, transposed + rotated + re-quantized out ---------------------------------
// in: codes [R, C/2], scales [R, C/32]; out: the [C, R] tensor quantized along R.
constexpr int kTileR = 128;
constexpr int kTileC = 128;

template <int VAL_DTYPE, int HD, int MODE>
__global__ __launch_bounds__(256) void requantize_transposed_kernel(const uint8_t* __restrict__ codes_in,
                                                                    const uint8_t* __restrict__ scales_in,
                                                                    int64_t R, int64_t C, float post, float c,
                                                                    SignBits sb, const float* __restrict__ u,
                                                                    uint64_t seed, QuantOut out) {
    constexpr int kPitch = kTileC / 2 / 4 + 1;  // dwords per row of packed codes (+1 pad)
    __shared__ uint32_t ctile[kTileR * kPitch];
    __shared__ uint32_t stile[kTileR];  // 4 scale bytes per row (128 columns)
    const int64_t r0 = (int64_t)blockIdx.x * kTileR;
    const int64_t c0 = (int64_t)blockIdx.y * kTileC;
    const int64_t code_pitch = C / 2, scale_pitch = C / 32;
    for (int idx = threadIdx.x; idx < kTileR * 4; idx += 256) {
        const int row = idx >> 2, cv = idx & 3;  // 4 x 16 B per row
        uint4 raw = make_uint4(0, 0, 0, 0);
        if (r0 + row < R && c0 + cv * 32 < C)
            raw = *reinterpret_cast<const uint4*>(codes_in + (r0 + row) * code_pitch + c0 / 2 + cv * 16);
        uint32_t* dst = ctile + row * kPitch + cv * 4;
        dst[0] = raw.x; dst[1] = raw.y; dst[2] = raw.z; dst[3] = raw.w;
    }
    if (threadIdx.x < kTileR) {
        const int row = threadIdx.x;
        uint32_t s = 0;
        if (r0 + row < R) {
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (c0 + b * 32 < C) s |= (uint32_t)scales_in[(r0 + row) * scale_pitch + c0 / 32 + b] << (8 * b);
        }
        stile[row] = s;
    }
    __syncthreads();
    constexpr int kOctPerC = kTileR / 8;
    for (int oc = threadIdx.x; oc < kTileC * kOctPerC; oc += 256) {
        const int cl = oc / kOctPerC, ro = oc % kOctPerC;
        if (r0 + ro * 8 >= R || c0 + cl >= C) continue;
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int row = ro * 8 + i;
            uint32_t w = ctile[row * kPitch + (cl >> 3)];
            uint32_t nib = (w >> (4 * (cl & 7))) & 15u;
            uint32_t sbyte = (stile[row] >> (8 * (cl >> 5))) & 0xffu;
            float q = e2m1_value((int)(nib & 7u));
            q = (nib & 8u) ? -q : q;
            float val = q * scale_pow2(post, (int)sbyte - 127);
            if constexpr (VAL_DTYPE == BF16) val = bf16_to_f32(f32_to_bf16(val));
            v[i] = val;
        }
        const int64_t octet = ((c0 + cl) * R + r0) / 8 + ro;
        using T = typename std::conditional<VAL_DTYPE == BF16, uint16_t, float>::type;
        process_octet<T, HD, MODE>(v, ro & (HD / 8 - 1), octet, c, sb, u, seed, out);
    }
}

template <typename T, int HD>
void launch_rowmajor(int mode, const void* x, int64_t n, float c, const SignBits& sb, const float* u, uint64_t seed,
                     const QuantOut& out, hipStream_t stream) {
    const int64_t n_octets = n / 8;
    dim3 grid((unsigned)((n_octets + 255) / 256)), block(256);
    const T* xp = reinterpret_cast<const T*>(x);
    switch (mode) {
        case QUEST_RTN: quantize_rowmajor_kernel<T, HD, QUEST_RTN><<<grid, block, 0, stream>>>(xp, n_octets, c, sb, u, seed, out); break;
        case ABSMAX_RTN: quantize_rowmajor_kernel<T, HD, ABSMAX_RTN><<<grid, block, 0, stream>>>(xp, n_octets, c, sb, u, seed, out); break;
        case ABSMAX_SR: quantize_rowmajor_kernel<T, HD, ABSMAX_SR><<<grid, block, 0, stream>>>(xp, n_octets, c, sb, u, seed, out); break;
        default: quantize_rowmajor_kernel<T, HD, QUEST_SR><<<grid, block, 0, stream>>>(xp, n_octets, c, sb, u, seed, out); break;
    }
}

template <typename T, int HD>
void launch_transposed(int mode, const void* x, int64_t P, int64_t Q, float c, const SignBits& sb, const float* u,
                       uint64_t seed, const QuantOut& out, hipStream_t stream) {
    dim3 grid((unsigned)((P + kTileP - 1) / kTileP), (unsigned)((Q + kTileQ - 1) / kTileQ)), block(256);
    const T* xp = reinterpret_cast<const T*>(x);
    switch (mode) {
        case QUEST_RTN: quantize_transposed_kernel<T, HD, QUEST_RTN><<<grid, block, 0, stream>>>(xp, P, Q, c, sb, u, seed, out); break;
        case ABSMAX_RTN: quantize_transposed_kernel<T, HD, ABSMAX_RTN><<<grid, block, 0, stream>>>(xp, P, Q, c, sb, u, seed, out); break;
        case ABSMAX_SR: quantize_transposed_kernel<T, HD, ABSMAX_SR><<<grid, block, 0, stream>>>(xp, P, Q, c, sb, u, seed, out); break;
        default: quantize_transposed_kernel<T, HD, QUEST_SR><<<grid, block, 0, stream>>>(xp, P, Q, c, sb, u, seed, out); break;
    }
}

template <int VAL_DTYPE, int HD>
void launch_requant(int mode, const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C, float post, float c,
                    const SignBits& sb, const float* u, uint64_t seed, const QuantOut& out, hipStream_t stream) {
    dim3 grid((unsigned)((R + kTileR - 1) / kTileR), (unsigned)((C + kTileC - 1) / kTileC)), block(256);
    switch (mode) {
        case QUEST_RTN: requantize_transposed_kernel<VAL_DTYPE, HD, QUEST_RTN><<<grid, block, 0, stream>>>(codes, scales, R, C, post, c, sb, u, seed, out); break;
        case ABSMAX_RTN: requantize_transposed_kernel<VAL_DTYPE, HD, ABSMAX_RTN><<<grid, block, 0, stream>>>(codes, scales, R, C, post, c, sb, u, seed, out); break;
        case ABSMAX_SR: requantize_transposed_kernel<VAL_DTYPE, HD, ABSMAX_SR><<<grid, block, 0, stream>>>(codes, scales, R, C, post, c, sb, u, seed, out); break;
        default: requantize_transposed_kernel<VAL_DTYPE, HD, QUEST_SR><<<grid, block, 0, stream>>>(codes, scales, R, C, post, c, sb, u, seed, out); break;
    }
}

template <typename F>
void dispatch_hd(int hd, F&& f) {
    if (hd == 32) f(std::integral_constant<int, 32>{});
    else if (hd == 64) f(std::integral_constant<int, 64>{});
    else f(std::integral_constant<int, 128>{});
}

}  // namespace

// The tiled code layout exists on the Hadamard-32 group-layout kernels only.
bool quantize_supports_tiled(int64_t rows, int64_t cols, int hd, int mode, bool transposed_in, const float* u,
                             const uint8_t* maskbits) {
    const bool rtn = (mode == QUEST_RTN || mode == ABSMAX_RTN);
    if (hd != 32 || !(rtn || u == nullptr) || rows % 16 || cols % 128) return false;
    return !transposed_in || maskbits == nullptr;
}
bool requantize_supports_tiled(int64_t R, int64_t C, int hd, int mode, const float* u) {
    const bool rtn = (mode == QUEST_RTN || mode == ABSMAX_RTN);
    return hd == 32 && (rtn || u == nullptr) && R % 128 == 0 && C % 128 == 0;
}

hipError_t quantize_mxfp4(const void* x, int dtype, int64_t rows, int64_t cols, int hd, const SignBits& sb, int mode,
                          bool transposed_in, const float* u, uint64_t seed, uint8_t* codes, uint8_t* scales,
                          uint8_t* maskbits, void* dequant, int codes_layout, hipStream_t stream) {
    if (rows == 0 || cols == 0) return hipSuccess;
    const bool rtn = (mode == QUEST_RTN || mode == ABSMAX_RTN);
    const bool tiled = codes_layout == LAYOUT_TILED;
    if (tiled && !quantize_supports_tiled(rows, cols, hd, mode, transposed_in, u, maskbits)) return hipErrorInvalidValue;
    const auto al = [](const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
    if (tiled && !(al(codes, 16) && al(maskbits, 4) && al(scales, 4))) return hipErrorInvalidValue;
    if (hd == 1) {
        // already rotated input: groups of 32 pass straight to the quantizer (row-major, RTN or seeded SR only)
        if (transposed_in || !(rtn || u == nullptr) || tiled || !al(codes, 16) || !al(maskbits, 4)) return hipErrorInvalidValue;
        return quantize_rowmajor_hd32(x, dtype, rows, cols, 0u, mode, seed, codes, scales, maskbits, dequant, false, false, stream);
    }
    if (hd == 32 && !transposed_in && (rtn || u == nullptr) && al(codes, 16) && al(maskbits, 4))
        return quantize_rowmajor_hd32(x, dtype, rows, cols, sb.w[0], mode, seed, codes, scales, maskbits, dequant, tiled, true, stream);
    if ((hd == 64 || hd == 128) && !transposed_in && (rtn || u == nullptr) && al(codes, 16) && al(maskbits, 4))
        return quantize_rowmajor_wide(x, dtype, rows * cols, hd, sb, mode, seed, codes, scales, maskbits, dequant, stream);
    // logical [rows, cols] = physical [P = cols, Q = rows]
    if (hd == 32 && transposed_in && (rtn || u == nullptr) && maskbits == nullptr && al(codes, 16) && al(scales, 4) &&
        cols % 128 == 0)
        return quantize_transposed_hd32(x, dtype, cols, rows, sb.w[0], mode, seed, codes, scales, dequant, tiled, stream);
    QuantOut out{reinterpret_cast<uint32_t*>(codes), scales, maskbits, dequant};
    const float c = hadamard_scale(hd, dtype);
    dispatch_hd(hd, [&](auto HDc) {
        constexpr int HD = decltype(HDc)::value;
        if (!transposed_in) {
            if (dtype == BF16) launch_rowmajor<uint16_t, HD>(mode, x, rows * cols, c, sb, u, seed, out, stream);
            else launch_rowmajor<float, HD>(mode, x, rows * cols, c, sb, u, seed, out, stream);
        } else {
            // logical [rows, cols] = physical [P = cols, Q = rows]
            if (dtype == BF16) launch_transposed<uint16_t, HD>(mode, x, cols, rows, c, sb, u, seed, out, stream);
            else launch_transposed<float, HD>(mode, x, cols, rows, c, sb, u, seed, out, stream);
        }
    });
    return hipGetLastError();
}

// Dense 32x32 rotation: served by the group-layout kernels only.  Row-major input: any rows, cols % 32 == 0.
// Transposed input (logical [rows, cols] = physical [cols, rows]): cols % 128 == 0, rows % 8 == 0, no clip mask.
hipError_t quantize_mxfp4_dense(const void* x, int dtype, int64_t rows, int64_t cols, const float* matrix, int mode,
                                bool transposed_in, uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits,
                                void* dequant, int codes_layout, hipStream_t stream) {
    if (rows == 0 || cols == 0) return hipSuccess;
    const bool tiled = codes_layout == LAYOUT_TILED;
    const auto al = [](const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
    if (!matrix || cols % 32 || !al(codes, 16) || !al(maskbits, 4) || !al(matrix, 4)) return hipErrorInvalidValue;
    if (tiled && (rows % 16 || cols % 128)) return hipErrorInvalidValue;
    if (!transposed_in)
        return quantize_rowmajor_dense(x, dtype, rows, cols, matrix, mode, seed, codes, scales, maskbits, dequant, tiled, stream);
    if (maskbits || cols % 128 || rows % 8 || !al(scales, 4)) return hipErrorInvalidValue;
    return quantize_transposed_dense(x, dtype, cols, rows, matrix, mode, seed, codes, scales, dequant, tiled, stream);
}

// R % 128 == 0, C % 32 == 0; tiled code bytes on either side need C % 128 == 0 as well
hipError_t requantize_transposed_mxfp4_dense(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C,
                                             float post, int val_dtype, const float* matrix, int mode, uint64_t seed,
                                             uint8_t* codes_out, uint8_t* scales_out, void* dequant, int in_layout,
                                             int out_layout, hipStream_t stream) {
    if (R == 0 || C == 0) return hipSuccess;
    const bool tiled_in = in_layout == LAYOUT_TILED, tiled_out = out_layout == LAYOUT_TILED;
    const auto al = [](const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
    if (!matrix || R % 128 || C % 32 || !al(codes_out, 16) || !al(scales_out, 4) || !al(codes_in, 16)) return hipErrorInvalidValue;
    if ((tiled_in || tiled_out) && C % 128) return hipErrorInvalidValue;
    return requantize_transposed_dense(codes_in, scales_in, R, C, post, val_dtype, matrix, mode, seed, codes_out, scales_out,
                                       dequant, tiled_in, tiled_out, stream);
}

hipError_t requantize_transposed_mxfp4(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C,
                                       float post, int val_dtype, int hd, const SignBits& sb, int mode, const float* u,
                                       uint64_t seed, uint8_t* codes_out, uint8_t* scales_out, void* dequant,
                                       int in_layout, int out_layout, hipStream_t stream) {
    if (R == 0 || C == 0) return hipSuccess;
    const bool rtn = (mode == QUEST_RTN || mode == ABSMAX_RTN);
    const bool tiled_in = in_layout == LAYOUT_TILED, tiled_out = out_layout == LAYOUT_TILED;
    const auto al = [](const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; };
    const bool fast = hd == 32 && (rtn || u == nullptr) && al(codes_out, 16) && al(scales_out, 4) && R % 128 == 0;
    if ((tiled_in || tiled_out) && !(fast && requantize_supports_tiled(R, C, hd, mode, u))) return hipErrorInvalidValue;
    if (fast)
        return requantize_transposed_hd32(codes_in, scales_in, R, C, post, val_dtype, sb.w[0], mode, seed, codes_out,
                                          scales_out, dequant, tiled_in, tiled_out, stream);
    QuantOut out{reinterpret_cast<uint32_t*>(codes_out), scales_out, nullptr, dequant};
    const float c = hadamard_scale(hd, val_dtype);
    dispatch_hd(hd, [&](auto HDc) {
        constexpr int HD = decltype(HDc)::value;
        if (val_dtype == BF16) launch_requant<BF16, HD>(mode, codes_in, scales_in, R, C, post, c, sb, u, seed, out, stream);
        else launch_requant<F32, HD>(mode, codes_in, scales_in, R, C, post, c, sb, u, seed, out, stream);
    });
    return hipGetLastError();
}

}  // namespace qm
