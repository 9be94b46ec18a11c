// MXFP4 x MXFP4 "TN" GEMM on gfx950's block-scaled FP4 MFMA (K2).
//
//   C[m, n] = alpha * sum_k A[m, k] * B[n, k]
//
// A: packed E2M1 codes [M, K/2] (element 2i in the low nibble of byte i) + E8M0 scales [M, K/32];
// B likewise with N rows.  Replaces the bf16 cuBLAS GEMMs the reference runs on de-quantized
// operands (src/models/quantization/backward.py:62,71-75,79-83) and the role of
// matmul_mxf4_bf16_tn in notebooks/benchmark_mxfp4.ipynb (CudaGemm).
//
// Instruction: v_mfma_scale_f32_32x32x64_f8f6f4 with both operands FP4.  Lane l of a wave feeds
// row (l % 32) of its operand with the 32 consecutive K values of one MX group (16 bytes) plus
// that group's E8M0 byte, so one MX group maps 1:1 onto one lane's share of the instruction.
// Within a K step of 128 (four MX groups per row) lane half h = l / 32 takes groups 2h and 2h+1
// in the two successive MFMAs; both operands use the same assignment, which is all the
// instruction needs.
//
// Tiling: workgroup = 4 waves, macro tile BM x BN, each wave owns a WM x WN block of 32x32 MFMA
// tiles with fp32 accumulators in registers.  Operands are staged global -> registers -> LDS
// (rows padded from 64 to 80 bytes so the 16-byte fragment reads of 16 consecutive rows hit 64
// distinct banks), double buffered, one barrier per K step.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qm_kernels.h"
#include "qm_math.h"

namespace qm {

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kBK = 128;             // K elements per step
constexpr int kRowBytes = kBK / 2;   // 64 bytes of codes per row per step
constexpr int kPitchDw = 20;         // 80-byte LDS row pitch, in dwords

template <int BM, int BN>
struct GemmSmem {
    static constexpr int kStageDw = (BM + BN) * kPitchDw + BM + BN;  // codes + one scale dword per row
    static constexpr int kBytes = 2 * kStageDw * 4;
};

__device__ __forceinline__ uint32_t load_scale_dword(const uint8_t* __restrict__ scales, int64_t row_pitch,
                                                     int64_t row, int64_t rows, int64_t g0, int64_t groups,
                                                     bool aligned) {
    if (row >= rows) return 0u;
    const uint8_t* p = scales + row * row_pitch + g0;
    if (aligned && g0 + 4 <= groups) return *reinterpret_cast<const uint32_t*>(p);
    uint32_t s = 0u;
#pragma unroll
    for (int b = 0; b < 4; ++b)
        if (g0 + b < groups) s |= (uint32_t)p[b] << (8 * b);
    return s;
}

template <int BM, int BN, int WM, int WN, typename OutT>
__global__ __launch_bounds__(256) void gemm_mxfp4_tn_kernel(const uint8_t* __restrict__ a_codes,
                                                            const uint8_t* __restrict__ a_scales,
                                                            const uint8_t* __restrict__ b_codes,
                                                            const uint8_t* __restrict__ b_scales, int64_t M,
                                                            int64_t N, int64_t K, float alpha,
                                                            OutT* __restrict__ c) {
    static_assert((BM / WM) * (BN / WN) == 4, "four waves per workgroup");
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int kAVec = BM * 4 / 256, kBVec = BN * 4 / 256;  // 16-byte loads per thread per step
    extern __shared__ uint32_t smem[];
    using S = GemmSmem<BM, BN>;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / (BN / WN), wn = wave % (BN / WN);
    const int lrow = lane & 31, half = lane >> 5;

    const int64_t m0 = (int64_t)blockIdx.y * BM, n0 = (int64_t)blockIdx.x * BN;
    const int64_t code_pitch = K / 2, groups = K / 32;
    const bool scales_aligned = (groups % 4) == 0;
    const int nk = (int)((K + kBK - 1) / kBK);

    uint4 ra[kAVec], rb[kBVec];
    uint32_t rs = 0u;

    auto load_global = [&](int ks) {
        const int64_t kbyte0 = (int64_t)ks * kRowBytes;
#pragma unroll
        for (int i = 0; i < kAVec; ++i) {
            const int idx = tid + i * 256, row = idx >> 2, cv = idx & 3;
            ra[i] = make_uint4(0, 0, 0, 0);
            if (m0 + row < M && kbyte0 + cv * 16 < code_pitch)
                ra[i] = *reinterpret_cast<const uint4*>(a_codes + (m0 + row) * code_pitch + kbyte0 + cv * 16);
        }
#pragma unroll
        for (int i = 0; i < kBVec; ++i) {
            const int idx = tid + i * 256, row = idx >> 2, cv = idx & 3;
            rb[i] = make_uint4(0, 0, 0, 0);
            if (n0 + row < N && kbyte0 + cv * 16 < code_pitch)
                rb[i] = *reinterpret_cast<const uint4*>(b_codes + (n0 + row) * code_pitch + kbyte0 + cv * 16);
        }
        // threads [0, BM) fetch A's scale dwords, threads [BM, BM+BN) fetch B's (BM + BN <= 512 -> two rounds)
        rs = 0u;
        if (tid < BM) rs = load_scale_dword(a_scales, groups, m0 + tid, M, (int64_t)ks * 4, groups, scales_aligned);
        else if (tid - BM < BN) rs = load_scale_dword(b_scales, groups, n0 + (tid - BM), N, (int64_t)ks * 4, groups, scales_aligned);
    };
    uint32_t rs2 = 0u;  // second round of scale rows when BM + BN > 256
    auto load_global_scales2 = [&](int ks) {
        if constexpr (BM + BN > 256) {
            const int t2 = tid + 256;
            rs2 = 0u;
            if (t2 < BM) rs2 = load_scale_dword(a_scales, groups, m0 + t2, M, (int64_t)ks * 4, groups, scales_aligned);
            else if (t2 - BM < BN) rs2 = load_scale_dword(b_scales, groups, n0 + (t2 - BM), N, (int64_t)ks * 4, groups, scales_aligned);
        }
    };
    auto store_lds = [&](int buf) {
        uint32_t* sa = smem + buf * S::kStageDw;
        uint32_t* sb = sa + BM * kPitchDw;
        uint32_t* ss = sb + BN * kPitchDw;  // [BM] A scales then [BN] B scales
#pragma unroll
        for (int i = 0; i < kAVec; ++i) {
            const int idx = tid + i * 256, row = idx >> 2, cv = idx & 3;
            *reinterpret_cast<uint4*>(sa + row * kPitchDw + cv * 4) = ra[i];
        }
#pragma unroll
        for (int i = 0; i < kBVec; ++i) {
            const int idx = tid + i * 256, row = idx >> 2, cv = idx & 3;
            *reinterpret_cast<uint4*>(sb + row * kPitchDw + cv * 4) = rb[i];
        }
        if (tid < BM + BN) ss[tid] = rs;
        if constexpr (BM + BN > 256) {
            if (tid + 256 < BM + BN) ss[tid + 256] = rs2;
        }
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    load_global(0);
    load_global_scales2(0);
    store_lds(0);
    __syncthreads();

    for (int ks = 0; ks < nk; ++ks) {
        const int buf = ks & 1;
        if (ks + 1 < nk) {
            load_global(ks + 1);
            load_global_scales2(ks + 1);
        }
        const uint32_t* sa = smem + buf * S::kStageDw;
        const uint32_t* sb = sa + BM * kPitchDw;
        const uint32_t* ss = sb + BN * kPitchDw;
        uint32_t sca[TM], scb[TN];
#pragma unroll
        for (int i = 0; i < TM; ++i) sca[i] = ss[wm * WM + i * 32 + lrow] >> (16 * half);
#pragma unroll
        for (int j = 0; j < TN; ++j) scb[j] = ss[BM + wn * WN + j * 32 + lrow] >> (16 * half);
#pragma unroll
        for (int sub = 0; sub < 2; ++sub) {
            v8i af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                uint4 q = *reinterpret_cast<const uint4*>(sa + (wm * WM + i * 32 + lrow) * kPitchDw + (2 * half + sub) * 4);
                af[i] = v8i{(int)q.x, (int)q.y, (int)q.z, (int)q.w, 0, 0, 0, 0};
            }
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                uint4 q = *reinterpret_cast<const uint4*>(sb + (wn * WN + j * 32 + lrow) * kPitchDw + (2 * half + sub) * 4);
                bf[j] = v8i{(int)q.x, (int)q.y, (int)q.z, (int)q.w, 0, 0, 0, 0};
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if (sub == 0)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[i], bf[j], acc[i][j], 4, 4, 0,
                                                                                     (int)sca[i], 0, (int)scb[j]);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(af[i], bf[j], acc[i][j], 4, 4, 1,
                                                                                     (int)sca[i], 1, (int)scb[j]);
                }
        }
        if (ks + 1 < nk) store_lds(buf ^ 1);
        __syncthreads();
    }

    // epilogue: acc element e of a 32x32 tile is row 8*(e/4) + 4*half + e%4, column lane%32
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int64_t col = n0 + wn * WN + j * 32 + lrow;
            if (col >= N) continue;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int64_t row = m0 + wm * WM + i * 32 + 8 * (e / 4) + 4 * half + (e & 3);
                if (row >= M) continue;
                const float v = acc[i][j][e] * alpha;
                if constexpr (sizeof(OutT) == 2) c[row * N + col] = f32_to_bf16(v);
                else c[row * N + col] = v;
            }
        }
}

template <int BM, int BN, int WM, int WN>
hipError_t launch_gemm(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                       const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype,
                       hipStream_t stream) {
    dim3 grid((unsigned)((N + BN - 1) / BN), (unsigned)((M + BM - 1) / BM)), block(256);
    constexpr int smem = GemmSmem<BM, BN>::kBytes;
    if (c_dtype == BF16) {
        auto kern = gemm_mxfp4_tn_kernel<BM, BN, WM, WN, uint16_t>;
        if (smem > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            if (e != hipSuccess) return e;
        }
        kern<<<grid, block, smem, stream>>>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, reinterpret_cast<uint16_t*>(c));
    } else {
        auto kern = gemm_mxfp4_tn_kernel<BM, BN, WM, WN, float>;
        if (smem > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, smem);
            if (e != hipSuccess) return e;
        }
        kern<<<grid, block, smem, stream>>>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, reinterpret_cast<float*>(c));
    }
    return hipGetLastError();
}

}  // namespace

hipError_t gemm_mxfp4_tn(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                         const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype,
                         hipStream_t stream) {
    if (M == 0 || N == 0) return hipSuccess;
    return launch_gemm<128, 128, 64, 64>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, c_dtype, stream);
}

}  // namespace qm
