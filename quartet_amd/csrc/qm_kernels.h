// Internal C++ entry points of the HIP kernels; the public C ABI (include/quartet_hip.h) wraps
// these after validating shapes.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace qm {

// bit j set = rotated column j is negated (H = c * S * diag(signs)); hd <= 128 columns
struct SignBits {
    uint32_t w[4];
};

hipError_t quantize_mxfp4(const void* x, int dtype, int64_t rows, int64_t cols, int hd, const SignBits& sb, int mode,
                          bool transposed_in, const float* u, uint64_t seed, uint8_t* codes, uint8_t* scales,
                          uint8_t* maskbits, void* dequant, hipStream_t stream);

// hd = 32 fast path (one MX group per lane, hardware FP4 converts); row-major input, RTN or Philox SR
hipError_t quantize_rowmajor_hd32(const void* x, int dtype, int64_t n, uint32_t sign_word, int mode, uint64_t seed,
                                  uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                                  hipStream_t stream);

hipError_t quantize_transposed_hd32(const void* x, int dtype, int64_t P, int64_t Q, uint32_t sign_word, int mode,
                                    uint64_t seed, uint8_t* codes, uint8_t* scales, void* dequant, hipStream_t stream);
hipError_t requantize_transposed_hd32(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C, float post,
                                      int val_dtype, uint32_t sign_word, int mode, uint64_t seed, uint8_t* codes,
                                      uint8_t* scales, void* dequant, hipStream_t stream);

hipError_t requantize_transposed_mxfp4(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C,
                                       float post, int val_dtype, int hd, const SignBits& sb, int mode, const float* u,
                                       uint64_t seed, uint8_t* codes_out, uint8_t* scales_out, void* dequant,
                                       hipStream_t stream);

hipError_t gemm_mxfp4_tn(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                         const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype,
                         hipStream_t stream);

hipError_t masked_hadamard_bwd(const void* g, int g_dtype, int64_t rows, int64_t cols, int hd, int scale_dtype,
                               const SignBits& sb, const uint8_t* maskbits, void* out, int out_dtype,
                               hipStream_t stream);

hipError_t dequantize_mxfp4(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C, float post, void* out,
                            int out_dtype, hipStream_t stream);

}  // namespace qm
