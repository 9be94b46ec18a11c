// C ABI of libquartet_hip.so: argument validation + dispatch to the kernels.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/quartet_hip.h"
#include "qm_kernels.h"

namespace {

thread_local char g_last_error[256] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
    va_end(ap);
    return code;
}

int from_hip(hipError_t e, const char* what) {
    if (e == hipSuccess) return 0;
    snprintf(g_last_error, sizeof(g_last_error), "%s: %s", what, hipGetErrorString(e));
    return (int)e;
}

bool aligned(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }
bool valid_hd(int hd) { return hd == 32 || hd == 64 || hd == 128; }
bool valid_dtype(int d) { return d == QM_BF16 || d == QM_F32; }
bool valid_mode(int m) { return m >= QM_QUEST_RTN && m <= QM_QUEST_SR; }
bool valid_layout(int l) { return l == QM_LAYOUT_ROWMAJOR || l == QM_LAYOUT_TILED; }

qm::SignBits make_signs(const uint32_t* sign_bits, int hd) {
    qm::SignBits sb{{0u, 0u, 0u, 0u}};
    if (sign_bits)
        for (int i = 0; i < (hd + 31) / 32; ++i) sb.w[i] = sign_bits[i];
    return sb;
}

}  // namespace

extern "C" {

int qm_version(void) { return 2; }

const char* qm_last_error(void) { return g_last_error; }

int qm_quantize_mxfp4(const void* x, int x_dtype, int64_t rows, int64_t cols, int hadamard_dim,
                      const uint32_t* sign_bits, int mode, int transposed_in, const float* u, uint64_t seed,
                      uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant, int codes_layout, void* stream) {
    if (!valid_layout(codes_layout)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: unknown codes_layout %d", codes_layout);
    if (!valid_dtype(x_dtype)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: x_dtype %d is not QM_BF16/QM_F32", x_dtype);
    if (!valid_hd(hadamard_dim)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: hadamard_dim %d not in {32,64,128}", hadamard_dim);
    if (!valid_mode(mode)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: unknown mode %d", mode);
    if (rows < 0 || cols < 0) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: negative shape [%lld, %lld]", (long long)rows, (long long)cols);
    if (cols % hadamard_dim) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: cols %lld not a multiple of hadamard_dim %d", (long long)cols, hadamard_dim);
    if (rows == 0 || cols == 0) return 0;
    if (!x || !codes || !scales) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: x, codes and scales must be non-null");
    if (transposed_in && rows % 8) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: transposed input needs rows %% 8 == 0 (got %lld)", (long long)rows);
    if (!aligned(x, 16) || !aligned(codes, 4) || (dequant && !aligned(dequant, 16)) || (u && !aligned(u, 16)))
        return fail(QM_ERR_UNALIGNED, "qm_quantize_mxfp4: x/dequant/u need 16-byte and codes 4-byte alignment");
    if (codes_layout == QM_LAYOUT_TILED &&
        (!qm::quantize_supports_tiled(rows, cols, hadamard_dim, mode, transposed_in != 0, u, maskbits) || !aligned(codes, 16) ||
         !aligned(scales, 4) || !aligned(maskbits, 4)))
        return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: tiled codes need hadamard_dim 32, rows %% 16 == 0, cols %% 128 == 0, "
                                    "no explicit uniforms, no mask with transposed input, 16-byte aligned codes (rows=%lld cols=%lld)",
                    (long long)rows, (long long)cols);
    return from_hip(qm::quantize_mxfp4(x, x_dtype, rows, cols, hadamard_dim, make_signs(sign_bits, hadamard_dim), mode,
                                       transposed_in != 0, u, seed, codes, scales, maskbits, dequant, codes_layout,
                                       reinterpret_cast<hipStream_t>(stream)),
                    "qm_quantize_mxfp4");
}

int qm_requantize_transposed_mxfp4(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C, float post,
                                   int val_dtype, int hadamard_dim, const uint32_t* sign_bits, int mode,
                                   const float* u, uint64_t seed, uint8_t* codes_out, uint8_t* scales_out,
                                   void* dequant, int in_layout, int out_layout, void* stream) {
    if (!valid_layout(in_layout) || !valid_layout(out_layout))
        return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4: unknown layout %d / %d", in_layout, out_layout);
    if (!valid_dtype(val_dtype)) return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4: val_dtype %d", val_dtype);
    if (!valid_hd(hadamard_dim)) return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4: hadamard_dim %d not in {32,64,128}", hadamard_dim);
    if (!valid_mode(mode)) return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4: unknown mode %d", mode);
    if (R < 0 || C < 0 || C % 32 || R % hadamard_dim)
        return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4: need C %% 32 == 0 and R %% hadamard_dim == 0 (R=%lld C=%lld hd=%d)", (long long)R, (long long)C, hadamard_dim);
    if (R == 0 || C == 0) return 0;
    if (!codes_in || !scales_in || !codes_out || !scales_out) return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4: null tensor");
    if (!aligned(codes_in, 16) || !aligned(codes_out, 4) || (dequant && !aligned(dequant, 16)) || (u && !aligned(u, 16)))
        return fail(QM_ERR_UNALIGNED, "qm_requantize_transposed_mxfp4: codes_in/dequant/u need 16-byte and codes_out 4-byte alignment");
    if ((in_layout == QM_LAYOUT_TILED || out_layout == QM_LAYOUT_TILED) &&
        (!qm::requantize_supports_tiled(R, C, hadamard_dim, mode, u) || !aligned(codes_out, 16) || !aligned(scales_out, 4)))
        return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4: tiled codes need hadamard_dim 32, R %% 128 == 0, C %% 128 == 0, "
                                    "no explicit uniforms, 16-byte aligned codes_out (R=%lld C=%lld)", (long long)R, (long long)C);
    return from_hip(qm::requantize_transposed_mxfp4(codes_in, scales_in, R, C, post, val_dtype, hadamard_dim,
                                                    make_signs(sign_bits, hadamard_dim), mode, u, seed, codes_out,
                                                    scales_out, dequant, in_layout, out_layout,
                                                    reinterpret_cast<hipStream_t>(stream)),
                    "qm_requantize_transposed_mxfp4");
}

int qm_gemm_mxfp4_tn(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                     int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype, int a_layout, int b_layout,
                     void* stream) {
    if (!valid_layout(a_layout) || !valid_layout(b_layout))
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: unknown layout %d / %d", a_layout, b_layout);
    if (!valid_dtype(c_dtype)) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: c_dtype %d", c_dtype);
    if (M < 0 || N < 0 || K < 0 || K % 32) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: need K %% 32 == 0 (M=%lld N=%lld K=%lld)", (long long)M, (long long)N, (long long)K);
    if (M == 0 || N == 0) return 0;
    if (!c || (K > 0 && (!a_codes || !a_scales || !b_codes || !b_scales))) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: null tensor");
    if (!aligned(a_codes, 16) || !aligned(b_codes, 16) || !aligned(a_scales, 4) || !aligned(b_scales, 4) || !aligned(c, 4))
        return fail(QM_ERR_UNALIGNED, "qm_gemm_mxfp4_tn: codes need 16-byte, scales and c 4-byte alignment");
    if ((a_layout == QM_LAYOUT_TILED || b_layout == QM_LAYOUT_TILED) && !qm::gemm_supports_tiled(M, N, K))
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: tiled operands need M %% 256 == 0, N %% 256 == 0, K %% 128 == 0 (M=%lld N=%lld K=%lld)",
                    (long long)M, (long long)N, (long long)K);
    return from_hip(qm::gemm_mxfp4_tn(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, c_dtype, a_layout, b_layout,
                                      reinterpret_cast<hipStream_t>(stream)),
                    "qm_gemm_mxfp4_tn");
}

int qm_masked_hadamard_bwd(const void* g, int g_dtype, int64_t rows, int64_t cols, int hadamard_dim, int scale_dtype,
                           const uint32_t* sign_bits, const uint8_t* maskbits, void* out, int out_dtype, void* stream) {
    if (!valid_dtype(g_dtype) || !valid_dtype(out_dtype) || !valid_dtype(scale_dtype))
        return fail(QM_ERR_INVALID, "qm_masked_hadamard_bwd: dtypes must be QM_BF16/QM_F32");
    if (!valid_hd(hadamard_dim)) return fail(QM_ERR_INVALID, "qm_masked_hadamard_bwd: hadamard_dim %d not in {32,64,128}", hadamard_dim);
    if (rows < 0 || cols < 0 || cols % hadamard_dim)
        return fail(QM_ERR_INVALID, "qm_masked_hadamard_bwd: cols %lld not a multiple of hadamard_dim %d", (long long)cols, hadamard_dim);
    if (rows == 0 || cols == 0) return 0;
    if (!g || !out) return fail(QM_ERR_INVALID, "qm_masked_hadamard_bwd: null tensor");
    if (!aligned(g, 16) || !aligned(out, 16)) return fail(QM_ERR_UNALIGNED, "qm_masked_hadamard_bwd: g and out need 16-byte alignment");
    return from_hip(qm::masked_hadamard_bwd(g, g_dtype, rows, cols, hadamard_dim, scale_dtype,
                                            make_signs(sign_bits, hadamard_dim), maskbits, out, out_dtype,
                                            reinterpret_cast<hipStream_t>(stream)),
                    "qm_masked_hadamard_bwd");
}

int qm_dequantize_mxfp4(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C, float post, void* out,
                        int out_dtype, void* stream) {
    if (!valid_dtype(out_dtype)) return fail(QM_ERR_INVALID, "qm_dequantize_mxfp4: out_dtype %d", out_dtype);
    if (R < 0 || C < 0 || C % 32) return fail(QM_ERR_INVALID, "qm_dequantize_mxfp4: need C %% 32 == 0 (R=%lld C=%lld)", (long long)R, (long long)C);
    if (R == 0 || C == 0) return 0;
    if (!codes || !scales || !out) return fail(QM_ERR_INVALID, "qm_dequantize_mxfp4: null tensor");
    if (!aligned(codes, 4) || !aligned(out, 16)) return fail(QM_ERR_UNALIGNED, "qm_dequantize_mxfp4: codes need 4-byte and out 16-byte alignment");
    return from_hip(qm::dequantize_mxfp4(codes, scales, R, C, post, out, out_dtype, reinterpret_cast<hipStream_t>(stream)),
                    "qm_dequantize_mxfp4");
}

}  // extern "C"
