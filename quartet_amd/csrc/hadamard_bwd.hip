// Straight-through backward of the forward quantizer and the MXFP4 de-quantizer.
//
// masked_hadamard_bwd replaces src/models/quantization/quantizers/mxfp4.py:143-146
//     grad_in = ((grad_out * mask).view(-1, hd)) @ H^T,   H = c * S * diag(signs)
// with the mask read as packed bits (bit i of byte j <-> element 8j+i).  Signs are applied to the
// input column, then the ascending-stride butterfly, then c: the same canonical order the forward
// rotation uses.  HBM traffic per element (bf16): 2 B in + 1/8 B mask + 2 B out.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "qm_jobs.h"
#include "qm_kernels.h"
#include "qm_math.h"

namespace qm {

namespace {

typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

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
    // lower lane of a butterfly: own + partner; upper lane: partner - own = partner + (-own)
    const uint32_t flip = (lane_in_chunk & LANE_MASK) ? 0x80000000u : 0u;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float p = lane_xor<LANE_MASK>(v[i]);
        v[i] = p + u2f(f2u(v[i]) ^ flip);
    }
}

// Eight values of one octet (already loaded into v) -> mask, sign flips, butterfly within the Hadamard block (whose other
// octets sit in the neighbouring lanes), c, store.  ROUND_OUT (fp32 out): the result is rounded to bf16 and then widened --
// what a bf16 result converted to fp32 afterwards holds, without the separate conversion pass.
template <typename TOut, int HD, bool ROUND_OUT>
__device__ __forceinline__ void rotate_octet(float (&v)[8], uint32_t keep, int64_t octet, float c, const SignBits& sb, TOut* __restrict__ out) {
    const int lic = (int)(octet & (HD / 8 - 1));
    const int j0 = lic * 8;
    const uint32_t sign8 = (sb.w[j0 >> 5] >> (j0 & 31)) & 0xffu;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        // g * mask as the reference multiplies: the factor is the float 1.0 or 0.0 built from the bit
        const uint32_t all = (uint32_t)__builtin_amdgcn_sbfe((int)keep, i, 1);  // 0 or ~0
        const float x = v[i] * u2f(all & 0x3f800000u);
        v[i] = u2f(f2u(x) ^ (((sign8 >> i) & 1u) << 31));
    }
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
    cross_lane_stage<1>(v, lic);
    cross_lane_stage<2>(v, lic);
    if constexpr (HD >= 64) cross_lane_stage<4>(v, lic);
    if constexpr (HD >= 128) cross_lane_stage<8>(v, lic);
    if constexpr (sizeof(TOut) == 2) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // v_cvt_pk_bf16_f32: round to nearest even, the same rounding as f32_to_bf16
            const v2bf p = __builtin_convertvector(v2f{v[2 * i] * c, v[2 * i + 1] * c}, v2bf);
            w[i] = __builtin_bit_cast(uint32_t, p);
        }
        *reinterpret_cast<uint4*>(out + octet * 8) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = v[i] * c;
        if constexpr (ROUND_OUT) {
#pragma unroll
            for (int i = 0; i < 8; i += 2) {
                const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[i], v[i + 1]}, v2bf));
                v[i] = u2f(w << 16);
                v[i + 1] = u2f(w & 0xffff0000u);
            }
        }
        *reinterpret_cast<float4*>(out + octet * 8) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(out + octet * 8 + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

// The work of one launch as a job (qm_jobs.h): two independent inverse rotations can share a grid.
// ROUND_IN (bf16 in, fp32 out): the result is rounded to bf16 before it is widened.
template <typename TIn, typename TOut, int HD, bool ROUND_IN = false>
struct HadamardBwdJob {
    const TIn* g;
    int64_t n_octets;
    float c;
    SignBits sb;
    const uint8_t* maskbits;
    TOut* out;
    unsigned blocks;

    HadamardBwdJob(const void* g_, int64_t n, float c_, const SignBits& sb_, const uint8_t* maskbits_, void* out_)
        : g(reinterpret_cast<const TIn*>(g_)), n_octets(n / 8), c(c_), sb(sb_), maskbits(maskbits_),
          out(reinterpret_cast<TOut*>(out_)), blocks((unsigned)((n / 8 + 255) / 256)) {}

    __device__ __forceinline__ void run(unsigned bid) const {
        const int64_t octet = (int64_t)bid * 256 + threadIdx.x;
        if (octet >= n_octets) return;
        float v[8];
        if constexpr (sizeof(TIn) == 2) {
            uint4 raw = *reinterpret_cast<const uint4*>(g + octet * 8);
            uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                v[2 * i] = u2f(w[i] << 16);
                v[2 * i + 1] = u2f(w[i] & 0xffff0000u);
            }
        } else {
            float4 a = *reinterpret_cast<const float4*>(g + octet * 8);
            float4 b = *reinterpret_cast<const float4*>(g + octet * 8 + 4);
            v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
            v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        }
        const uint32_t keep = maskbits ? (uint32_t)maskbits[octet] : 0xffu;
        job_requests_issued();
        rotate_octet<TOut, HD, ROUND_IN>(v, keep, octet, c, sb, out);
    }
};

// The same rotation on a product that was cut into K ranges: the input element is alpha * (p[0][i] + p[1][i] + ...)
// summed in slab order (what the ordered reduction of the partial sums stores), rounded to bf16 when the product's own
// dtype is bf16 (MID_BF16).  One pass in place of the reduction followed by the rotation, with the same arithmetic.
template <bool MID_BF16, typename TOut>
struct SplitKRotateJob {
    const float* partial;
    int splits;
    int64_t mn;
    float alpha, c;
    SignBits sb;
    const uint8_t* maskbits;
    TOut* out;
    unsigned blocks;

    SplitKRotateJob(const float* partial_, int splits_, int64_t mn_, float alpha_, float c_, const SignBits& sb_, const uint8_t* maskbits_,
                    void* out_)
        : partial(partial_), splits(splits_), mn(mn_), alpha(alpha_), c(c_), sb(sb_), maskbits(maskbits_),
          out(reinterpret_cast<TOut*>(out_)), blocks((unsigned)((mn_ / 8 + 255) / 256)) {}

    __device__ __forceinline__ void run(unsigned bid) const {
        const int64_t octet = (int64_t)bid * 256 + threadIdx.x;
        if (octet >= mn / 8) return;
        const float* p = partial + octet * 8;
        float4 a = *reinterpret_cast<const float4*>(p);
        float4 b = *reinterpret_cast<const float4*>(p + 4);
        const uint32_t keep = (uint32_t)maskbits[octet];
        for (int s = 1; s < splits; ++s) {
            const float4 x = *reinterpret_cast<const float4*>(p + (int64_t)s * mn);
            const float4 y = *reinterpret_cast<const float4*>(p + (int64_t)s * mn + 4);
            a.x += x.x; a.y += x.y; a.z += x.z; a.w += x.w;
            b.x += y.x; b.y += y.y; b.z += y.z; b.w += y.w;
        }
        job_requests_issued();
        float v[8] = {a.x * alpha, a.y * alpha, a.z * alpha, a.w * alpha, b.x * alpha, b.y * alpha, b.z * alpha, b.w * alpha};
        if constexpr (MID_BF16) {
#pragma unroll
            for (int i = 0; i < 8; ++i) v[i] = u2f((uint32_t)f32_to_bf16(v[i]) << 16);
        }
        rotate_octet<TOut, 32, MID_BF16 && sizeof(TOut) == 4>(v, keep, octet, c, sb, out);
    }
};

template <typename TOut>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint32_t* __restrict__ codes,
                                                         const uint8_t* __restrict__ scales, int64_t n_octets,
                                                         float post, TOut* __restrict__ out) {
    const int64_t octet = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (octet >= n_octets) return;
    const uint32_t w = codes[octet];
    const float scale = scale_pow2(post, (int)scales[octet >> 2] - 127);
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint32_t nib = (w >> (4 * i)) & 15u;
        float q = e2m1_value((int)(nib & 7u));
        v[i] = ((nib & 8u) ? -q : q) * scale;
    }
    if constexpr (sizeof(TOut) == 2) {
        uint32_t o[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = (uint32_t)f32_to_bf16(v[2 * i]) | ((uint32_t)f32_to_bf16(v[2 * i + 1]) << 16);
        *reinterpret_cast<uint4*>(out + octet * 8) = make_uint4(o[0], o[1], o[2], o[3]);
    } else {
        *reinterpret_cast<float4*>(out + octet * 8) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(out + octet * 8 + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
}

template <typename TIn, typename TOut, bool ROUND_IN = false>
void launch_bwd(int hd, const void* g, int64_t n, float c, const SignBits& sb, const uint8_t* maskbits, void* out,
                hipStream_t stream) {
    const auto go = [&](auto job) { launch_job(job, stream); };
    if (hd == 32) go(HadamardBwdJob<TIn, TOut, 32, ROUND_IN>(g, n, c, sb, maskbits, out));
    else if (hd == 64) go(HadamardBwdJob<TIn, TOut, 64, ROUND_IN>(g, n, c, sb, maskbits, out));
    else go(HadamardBwdJob<TIn, TOut, 128, ROUND_IN>(g, n, c, sb, maskbits, out));
}

}  // namespace

// round_to_g_dtype: with bf16 g and fp32 out, round the result to bf16 before widening
hipError_t masked_hadamard_bwd(const void* g, int g_dtype, int64_t rows, int64_t cols, int hd, int scale_dtype,
                               const SignBits& sb, const uint8_t* maskbits, void* out, int out_dtype,
                               bool round_to_g_dtype, hipStream_t stream) {
    if (rows == 0 || cols == 0) return hipSuccess;
    const float c = hadamard_scale(hd, scale_dtype);
    const int64_t n = rows * cols;
    if (g_dtype == BF16 && out_dtype == BF16) launch_bwd<uint16_t, uint16_t>(hd, g, n, c, sb, maskbits, out, stream);
    else if (g_dtype == BF16 && round_to_g_dtype) launch_bwd<uint16_t, float, true>(hd, g, n, c, sb, maskbits, out, stream);
    else if (g_dtype == BF16) launch_bwd<uint16_t, float>(hd, g, n, c, sb, maskbits, out, stream);
    else if (out_dtype == BF16) launch_bwd<float, uint16_t>(hd, g, n, c, sb, maskbits, out, stream);
    else launch_bwd<float, float>(hd, g, n, c, sb, maskbits, out, stream);
    return hipGetLastError();
}

// two independent masked inverse rotations (Hadamard block 32, element type `dtype` in; a out in `dtype`, b out in
// out_dtype_b: `dtype`, or fp32 holding the bf16-rounded result) in one grid
hipError_t masked_hadamard_bwd_hd32_pair(const void* ga, int64_t na, int scale_dtype_a, uint32_t sign_a, const uint8_t* mask_a, void* out_a,
                                         const void* gb, int64_t nb, int scale_dtype_b, uint32_t sign_b, const uint8_t* mask_b, void* out_b,
                                         int dtype, int out_dtype_b, hipStream_t stream) {
    const SignBits sa{{sign_a, 0, 0, 0}}, sb{{sign_b, 0, 0, 0}};
    const float ca = hadamard_scale(32, scale_dtype_a), cb = hadamard_scale(32, scale_dtype_b);
    if (dtype == BF16 && out_dtype_b == F32) {
        launch_job_pair(HadamardBwdJob<uint16_t, uint16_t, 32>(ga, na, ca, sa, mask_a, out_a),
                        HadamardBwdJob<uint16_t, float, 32, true>(gb, nb, cb, sb, mask_b, out_b), stream);
    } else if (dtype == BF16) {
        using J = HadamardBwdJob<uint16_t, uint16_t, 32>;
        launch_job_pair(J(ga, na, ca, sa, mask_a, out_a), J(gb, nb, cb, sb, mask_b, out_b), stream);
    } else {
        using J = HadamardBwdJob<float, float, 32>;
        launch_job_pair(J(ga, na, ca, sa, mask_a, out_a), J(gb, nb, cb, sb, mask_b, out_b), stream);
    }
    return hipGetLastError();
}

// c = masked inverse rotation (blocks of 32 along the rows) of the reduced product alpha * sum_s partial[s]; see SplitKRotateJob
hipError_t splitk_reduce_rotated(const float* partial, int splits, int64_t mn, float alpha, int mid_dtype, const uint8_t* maskbits,
                                 uint32_t sign_word, int scale_dtype, void* out, int out_dtype, hipStream_t stream) {
    if (mn == 0) return hipSuccess;
    if (mn % 32 || !maskbits || splits < 1 || (mid_dtype == F32 && out_dtype != F32)) return hipErrorInvalidValue;
    const SignBits sb{{sign_word, 0, 0, 0}};
    const float c = hadamard_scale(32, scale_dtype);
    if (mid_dtype == BF16 && out_dtype == BF16) launch_job(SplitKRotateJob<true, uint16_t>(partial, splits, mn, alpha, c, sb, maskbits, out), stream);
    else if (mid_dtype == BF16) launch_job(SplitKRotateJob<true, float>(partial, splits, mn, alpha, c, sb, maskbits, out), stream);
    else launch_job(SplitKRotateJob<false, float>(partial, splits, mn, alpha, c, sb, maskbits, out), stream);
    return hipGetLastError();
}

hipError_t dequantize_mxfp4(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C, float post, void* out,
                            int out_dtype, hipStream_t stream) {
    if (R == 0 || C == 0) return hipSuccess;
    const int64_t n_octets = R * C / 8;
    dim3 grid((unsigned)((n_octets + 255) / 256)), block(256);
    if (out_dtype == BF16)
        dequantize_kernel<uint16_t><<<grid, block, 0, stream>>>(reinterpret_cast<const uint32_t*>(codes), scales, n_octets, post, reinterpret_cast<uint16_t*>(out));
    else
        dequantize_kernel<float><<<grid, block, 0, stream>>>(reinterpret_cast<const uint32_t*>(codes), scales, n_octets, post, reinterpret_cast<float*>(out));
    return hipGetLastError();
}

}  // namespace qm
