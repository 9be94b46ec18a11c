// C ABI of libquartet_hip.so: argument validation + dispatch to the kernels.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include <mutex>

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

int qm_version(void) { return 15; }

const char* qm_last_error(void) { return g_last_error; }

int qm_quantize_mxfp4(const void* x, int x_dtype, int64_t rows, int64_t cols, int hadamard_dim,
                      const uint32_t* sign_bits, int mode, int transposed_in, const float* u, uint64_t seed,
                      uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant, int codes_layout, void* stream) {
    if (!valid_layout(codes_layout)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: unknown codes_layout %d", codes_layout);
    if (!valid_dtype(x_dtype)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: x_dtype %d is not QM_BF16/QM_F32", x_dtype);
    if (!valid_hd(hadamard_dim) && hadamard_dim != 1)
        return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: hadamard_dim %d not in {1,32,64,128}", hadamard_dim);
    if (hadamard_dim == 1 && (transposed_in || u || sign_bits || codes_layout != QM_LAYOUT_ROWMAJOR || cols % 32 ||
                              !aligned(codes, 16) || !aligned(maskbits, 4)))
        return fail(QM_ERR_INVALID, "qm_quantize_mxfp4: hadamard_dim 1 (input already rotated) needs row-major input and codes, "
                                    "cols %% 32 == 0, no sign bits, no explicit uniforms, 16-byte aligned codes");
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

int qm_quantize_mxfp4_dense(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* matrix, int mode,
                            int transposed_in, uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                            int codes_layout, void* stream) {
    if (!valid_layout(codes_layout)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4_dense: unknown codes_layout %d", codes_layout);
    if (!valid_dtype(x_dtype)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4_dense: x_dtype %d is not QM_BF16/QM_F32", x_dtype);
    if (!valid_mode(mode)) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4_dense: unknown mode %d", mode);
    if (rows < 0 || cols < 0 || cols % 32)
        return fail(QM_ERR_INVALID, "qm_quantize_mxfp4_dense: cols %lld not a multiple of 32", (long long)cols);
    if (rows == 0 || cols == 0) return 0;
    if (!x || !codes || !scales || !matrix) return fail(QM_ERR_INVALID, "qm_quantize_mxfp4_dense: x, matrix, codes and scales must be non-null");
    if (!aligned(x, 16) || !aligned(codes, 16) || !aligned(matrix, 4) || !aligned(maskbits, 4) || (dequant && !aligned(dequant, 16)))
        return fail(QM_ERR_UNALIGNED, "qm_quantize_mxfp4_dense: x/codes/dequant need 16-byte, matrix and maskbits 4-byte alignment");
    if (transposed_in && (maskbits || cols % 128 || rows % 8 || !aligned(scales, 4)))
        return fail(QM_ERR_INVALID, "qm_quantize_mxfp4_dense: transposed input needs cols %% 128 == 0, rows %% 8 == 0, no clip mask, "
                                    "4-byte aligned scales (rows=%lld cols=%lld)", (long long)rows, (long long)cols);
    if (codes_layout == QM_LAYOUT_TILED && (rows % 16 || cols % 128))
        return fail(QM_ERR_INVALID, "qm_quantize_mxfp4_dense: tiled codes need rows %% 16 == 0 and cols %% 128 == 0 (rows=%lld cols=%lld)",
                    (long long)rows, (long long)cols);
    return from_hip(qm::quantize_mxfp4_dense(x, x_dtype, rows, cols, matrix, mode, transposed_in != 0, seed, codes, scales, maskbits,
                                             dequant, codes_layout, reinterpret_cast<hipStream_t>(stream)),
                    "qm_quantize_mxfp4_dense");
}

int qm_requantize_transposed_mxfp4_dense(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C, float post,
                                         int val_dtype, const float* matrix, int mode, uint64_t seed, uint8_t* codes_out,
                                         uint8_t* scales_out, void* dequant, int in_layout, int out_layout, void* stream) {
    if (!valid_layout(in_layout) || !valid_layout(out_layout))
        return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4_dense: unknown layout %d / %d", in_layout, out_layout);
    if (!valid_dtype(val_dtype)) return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4_dense: val_dtype %d", val_dtype);
    if (!valid_mode(mode)) return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4_dense: unknown mode %d", mode);
    if (R < 0 || C < 0 || C % 32 || R % 128)
        return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4_dense: need C %% 32 == 0 and R %% 128 == 0 (R=%lld C=%lld)", (long long)R, (long long)C);
    if (R == 0 || C == 0) return 0;
    if (!codes_in || !scales_in || !codes_out || !scales_out || !matrix) return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4_dense: null tensor");
    if (!aligned(codes_in, 16) || !aligned(codes_out, 16) || !aligned(scales_out, 4) || !aligned(matrix, 4) || (dequant && !aligned(dequant, 16)))
        return fail(QM_ERR_UNALIGNED, "qm_requantize_transposed_mxfp4_dense: codes and dequant need 16-byte, scales_out and matrix 4-byte alignment");
    if ((in_layout == QM_LAYOUT_TILED || out_layout == QM_LAYOUT_TILED) && C % 128)
        return fail(QM_ERR_INVALID, "qm_requantize_transposed_mxfp4_dense: tiled codes need C %% 128 == 0 (C=%lld)", (long long)C);
    return from_hip(qm::requantize_transposed_mxfp4_dense(codes_in, scales_in, R, C, post, val_dtype, matrix, mode, seed, codes_out,
                                                          scales_out, dequant, in_layout, out_layout,
                                                          reinterpret_cast<hipStream_t>(stream)),
                    "qm_requantize_transposed_mxfp4_dense");
}

int qm_gemm_mxfp4_tn(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                     int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype, int a_layout, int b_layout,
                     void* workspace, size_t workspace_bytes, void* stream) {
    if (!valid_layout(a_layout) || !valid_layout(b_layout))
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: unknown layout %d / %d", a_layout, b_layout);
    if (!valid_dtype(c_dtype)) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: c_dtype %d", c_dtype);
    if (M < 0 || N < 0 || K < 0 || K % 32) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: need K %% 32 == 0 (M=%lld N=%lld K=%lld)", (long long)M, (long long)N, (long long)K);
    if (M == 0 || N == 0) return 0;
    if (!c || (K > 0 && (!a_codes || !a_scales || !b_codes || !b_scales))) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: null tensor");
    // the 256 x 256 tile kernels store c in 16-byte pieces; the generic kernel (any M, N) stores single elements
    const uintptr_t c_align = qm::gemm_supports_tiled(M, N, K) ? 16 : 4;
    if (!aligned(a_codes, 16) || !aligned(b_codes, 16) || !aligned(a_scales, 4) || !aligned(b_scales, 4) || !aligned(c, c_align))
        return fail(QM_ERR_UNALIGNED, "qm_gemm_mxfp4_tn: codes need 16-byte, scales 4-byte alignment, c 16-byte (4-byte for shapes "
                                      "outside the tile kernels: M or N not a multiple of 64 or below 256, K %% 128 != 0)");
    if ((a_layout == QM_LAYOUT_TILED || b_layout == QM_LAYOUT_TILED) && !qm::gemm_supports_tiled(M, N, K))
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn: tiled operands need M, N multiples of 64 and >= 256, K %% 128 == 0 (M=%lld N=%lld K=%lld)",
                    (long long)M, (long long)N, (long long)K);
    return from_hip(qm::gemm_mxfp4_tn(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, c_dtype, a_layout, b_layout,
                                      workspace, workspace_bytes, reinterpret_cast<hipStream_t>(stream)),
                    "qm_gemm_mxfp4_tn");
}

int qm_diag_gemm_tile_phases(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                             int64_t M, int64_t N, int64_t K, float alpha, void* c, int a_layout, int b_layout,
                             const uint8_t* maskbits, uint64_t* stamps, size_t stamps_bytes, void* stream) {
    if (!a_codes || !a_scales || !b_codes || !b_scales || !c || !stamps || !aligned(a_codes, 16) || !aligned(b_codes, 16) ||
        !aligned(c, 16) || !aligned(stamps, 8) || !aligned(maskbits, 4) || !valid_layout(a_layout) || !valid_layout(b_layout))
        return fail(QM_ERR_INVALID, "qm_diag_gemm_tile_phases: null, misaligned or ill-typed arguments");
    int grid = 0;
    const hipError_t e = qm::gemm_tile_phases(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, a_layout, b_layout, maskbits,
                                              reinterpret_cast<unsigned long long*>(stamps), stamps_bytes, &grid,
                                              reinterpret_cast<hipStream_t>(stream));
    if (e == hipErrorInvalidValue && grid == 0)
        return fail(QM_ERR_INVALID, "qm_diag_gemm_tile_phases: serves M, N multiples of 64 and >= 256, K %% 512 == 0, 16-byte aligned scales, "
                                    "and needs %d 64-bit values per workgroup in stamps", qm::gemm_phase_stamps_per_group());
    if (int rc = from_hip(e, "qm_diag_gemm_tile_phases")) return rc > 0 ? -rc : rc;
    return grid;
}

int64_t qm_diag_mfma_only(const uint8_t* operands, size_t operand_bytes, float* sink, size_t sink_bytes, int iters, void* stream) {
    const int blocks = qm::mfma_only_blocks();
    if (!operands || !sink || iters < 0 || operand_bytes < (size_t)blocks * 32768 || sink_bytes < (size_t)blocks * 1024 ||
        !aligned(operands, 16) || !aligned(sink, 4))
        return fail(QM_ERR_INVALID, "qm_diag_mfma_only: needs %zu bytes of operands (16-byte aligned) and %zu bytes of sink",
                    (size_t)blocks * 32768, (size_t)blocks * 1024);
    if (int rc = from_hip(qm::mfma_only(operands, sink, iters, reinterpret_cast<hipStream_t>(stream)), "qm_diag_mfma_only")) return -(int64_t)(rc > 0 ? rc : -rc);
    return (int64_t)blocks * 4 * (int64_t)iters * 16;
}

int qm_gemm_mxfp4_bf16_nn(const uint8_t* a_codes, const uint8_t* a_scales, const void* b, int64_t M, int64_t N, int64_t K,
                          float alpha, void* c, int c_dtype, void* stream) {
    if (!valid_dtype(c_dtype)) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_bf16_nn: c_dtype %d", c_dtype);
    if (M < 0 || N < 0 || K < 0) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_bf16_nn: negative extent");
    if (M == 0 || N == 0) return 0;
    if (!qm::gemm_fp4_bf16_nn_supported(M, N, K))
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_bf16_nn: need K a positive multiple of 64 and N a multiple of 8 (M=%lld N=%lld K=%lld)",
                    (long long)M, (long long)N, (long long)K);
    if (!a_codes || !a_scales || !b || !c) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_bf16_nn: null tensor");
    if (!aligned(a_codes, 16) || !aligned(a_scales, 2) || !aligned(b, 16) || !aligned(c, 16))
        return fail(QM_ERR_UNALIGNED, "qm_gemm_mxfp4_bf16_nn: a_codes, b and c need 16-byte, a_scales 2-byte alignment");
    return from_hip(qm::gemm_fp4_bf16_nn(a_codes, a_scales, b, M, N, K, alpha, c, c_dtype, reinterpret_cast<hipStream_t>(stream)),
                    "qm_gemm_mxfp4_bf16_nn");
}

size_t qm_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % 32) return 0;
    return qm::gemm_workspace_bytes(M, N, K);
}

}  // extern "C"

// ---- the product without any allocation: split-K partial sums live in a file-scope device array ---------------
namespace {
constexpr size_t kNoAllocScratchBytes = QM_GEMM_NOALLOC_SCRATCH_BYTES;
// One copy per GPU the library is loaded on, held until the process ends.  In host code this name is only a handle for
// hipGetSymbolAddress: the device address of each GPU's copy is looked up once per device and used from then on.
static __device__ __align__(256) __attribute__((used)) unsigned char scratch[kNoAllocScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// device address of the current device's scratch array (nullptr + error code on failure)
int scratch_of_current_device(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return from_hip(e, "qm_gemm_mxfp4_tn_noalloc: hipGetDevice");
    if (dev < 0 || dev >= kMaxDevices) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_noalloc: device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return from_hip(e == hipSuccess ? hipErrorInvalidSymbol : e, "qm_gemm_mxfp4_tn_noalloc: hipGetSymbolAddress");
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return 0;
}
}  // namespace

extern "C" {

size_t qm_gemm_noalloc_scratch_bytes(void) { return kNoAllocScratchBytes; }

int qm_gemm_noalloc_prepare(void) {
    void* ws = nullptr;
    return scratch_of_current_device(&ws);
}

int qm_gemm_mxfp4_tn_noalloc(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                             int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype, int a_layout, int b_layout,
                             void* stream) {
    if (M < 0 || N < 0 || K < 0 || K % 32)
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_noalloc: need K %% 32 == 0 (M=%lld N=%lld K=%lld)", (long long)M, (long long)N, (long long)K);
    if (M == 0 || N == 0) return 0;
    // the same cut into K ranges as qm_gemm_mxfp4_tn makes when it is offered qm_gemm_workspace_bytes() of scratch
    const size_t need = qm::gemm_workspace_bytes(M, N, K);
    if (need > kNoAllocScratchBytes)
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_noalloc: this shape's split-K partial sums need %zu bytes, the built-in scratch "
                                    "holds %zu (M=%lld N=%lld K=%lld); use qm_gemm_mxfp4_tn with a caller-provided workspace",
                    need, kNoAllocScratchBytes, (long long)M, (long long)N, (long long)K);
    // resolved on every path, so that the first call on a device is the only one that can make the runtime load this
    // library's device image (qm_gemm_noalloc_prepare() does the same ahead of time)
    void* ws = nullptr;
    if (int rc = scratch_of_current_device(&ws)) return rc;
    return qm_gemm_mxfp4_tn(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, c_dtype, a_layout, b_layout, need ? ws : nullptr, need, stream);
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
                                            make_signs(sign_bits, hadamard_dim), maskbits, out, out_dtype, false,
                                            reinterpret_cast<hipStream_t>(stream)),
                    "qm_masked_hadamard_bwd");
}

int qm_gemm_fuses_rotation(const uint8_t* a_scales, const uint8_t* b_scales, int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0 || K % 32) return 0;
    // offered the workspace the plain product would use: a shape it would cut into K ranges is not served
    const size_t ws = qm::gemm_workspace_bytes(M, N, K);
    return ws == 0 && qm::gemm_will_rotate(a_scales, b_scales, M, N, K, QM_BF16, QM_BF16, nullptr, 0) ? 1 : 0;
}

int qm_gemm_mxfp4_tn_rotated(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                             int64_t M, int64_t N, int64_t K, float alpha, void* c, int a_layout, int b_layout,
                             const uint8_t* maskbits, const uint32_t* sign_bits, int scale_dtype, void* stream) {
    if (!valid_layout(a_layout) || !valid_layout(b_layout))
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_rotated: unknown layout %d / %d", a_layout, b_layout);
    if (!valid_dtype(scale_dtype)) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_rotated: scale_dtype %d", scale_dtype);
    if (M < 0 || N < 0 || K < 0) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_rotated: negative extent");
    if (M == 0 || N == 0) return 0;
    if (!c || !a_codes || !a_scales || !b_codes || !b_scales || !maskbits) return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_rotated: null tensor");
    if (!qm_gemm_fuses_rotation(a_scales, b_scales, M, N, K))
        return fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_rotated: shape M=%lld N=%lld K=%lld is not served with the rotation fused "
                                    "(see qm_gemm_fuses_rotation); call qm_gemm_mxfp4_tn and qm_masked_hadamard_bwd",
                    (long long)M, (long long)N, (long long)K);
    if (!aligned(a_codes, 16) || !aligned(b_codes, 16) || !aligned(a_scales, 4) || !aligned(b_scales, 4) || !aligned(c, 16) || !aligned(maskbits, 4))
        return fail(QM_ERR_UNALIGNED, "qm_gemm_mxfp4_tn_rotated: codes and c need 16-byte, scales and mask bits 4-byte alignment");
    bool rotated = false;
    const int rc = from_hip(qm::gemm_mxfp4_tn_rotated(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, QM_BF16, a_layout, b_layout,
                                                      nullptr, 0, maskbits, sign_bits ? sign_bits[0] : 0u, scale_dtype, QM_BF16, &rotated,
                                                      reinterpret_cast<hipStream_t>(stream)), "qm_gemm_mxfp4_tn_rotated");
    if (rc) return rc;
    return rotated ? 0 : fail(QM_ERR_INVALID, "qm_gemm_mxfp4_tn_rotated: the product did not run as planned");
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


// ---- whole-layer entry points: one call issues every launch of the forward / backward pass -------------------

namespace {
size_t up256(size_t v) { return (v + 255) & ~(size_t)255; }
size_t esize(int dtype) { return dtype == QM_BF16 ? 2 : 4; }

// one packed operand: codes, scales, mask bits, each region 256-byte aligned
struct PackedLayout {
    size_t c, s, m, total;
};
PackedLayout packed_layout(int64_t rows, int64_t cols) {
    PackedLayout l;
    size_t o = 0;
    l.c = o; o += up256((size_t)rows * cols / 2);
    l.s = o; o += up256((size_t)rows * cols / 32);
    l.m = o; o += up256((size_t)rows * cols / 8);
    l.total = o;
    return l;
}
struct WorkLayout {
    size_t ec, es, wtc, wts, gxq, etc, ets, xtc, xts, gwq, gemm_ws, gemm_ws_bytes, total;
};
WorkLayout work_layout(int64_t T, int64_t I, int64_t O, int mid_dtype) {
    WorkLayout l;
    size_t o = 0;
    l.ec = o; o += up256((size_t)T * O / 2);
    l.es = o; o += up256((size_t)T * O / 32);
    l.wtc = o; o += up256((size_t)I * O / 2);
    l.wts = o; o += up256((size_t)I * O / 32);
    l.gxq = o; o += up256((size_t)T * I * esize(mid_dtype));
    l.etc = o; o += up256((size_t)O * T / 2);
    l.ets = o; o += up256((size_t)O * T / 32);
    l.xtc = o; o += up256((size_t)I * T / 2);
    l.xts = o; o += up256((size_t)I * T / 32);
    l.gwq = o; o += up256((size_t)O * I * esize(mid_dtype));
    const size_t g1 = qm::gemm_workspace_bytes(T, I, O), g2 = qm::gemm_workspace_bytes(O, I, T);
    l.gemm_ws_bytes = g1 > g2 ? g1 : g2;  // split-K scratch, shared by the two products (they run one after the other)
    l.gemm_ws = o; o += up256(l.gemm_ws_bytes);
    l.total = o;
    return l;
}
// The whole-layer calls issue independent launches two to a grid when all of them run on the Hadamard-32 kernels with
// tiled codes (which needs every extent to be a multiple of 128).
bool pair_launches(int codes_layout, int64_t T, int64_t I, int64_t O, int hd_a, int hd_b, int hd_c) {
    return codes_layout == QM_LAYOUT_TILED && hd_a == 32 && hd_b == 32 && hd_c == 32 && T % 128 == 0 && I % 128 == 0 &&
           O % 128 == 0;
}
}  // namespace

size_t qm_packed_operand_bytes(int64_t rows, int64_t cols) {
    if (rows < 0 || cols < 0 || cols % 32) return 0;
    return packed_layout(rows, cols).total;
}

int qm_packed_operand_offsets(int64_t rows, int64_t cols, size_t* offsets) {
    if (rows < 0 || cols < 0 || cols % 32 || !offsets)
        return fail(QM_ERR_INVALID, "qm_packed_operand_offsets: need cols %% 32 == 0 and a non-null array (rows=%lld cols=%lld)",
                    (long long)rows, (long long)cols);
    const PackedLayout l = packed_layout(rows, cols);
    offsets[0] = l.c; offsets[1] = l.s; offsets[2] = l.m;
    return 0;
}

size_t qm_linear_backward_workspace_bytes(int64_t T, int64_t I, int64_t O, int mid_dtype) {
    if (T < 0 || I < 0 || O < 0 || I % 32 || O % 32 || T % 32 || !valid_dtype(mid_dtype)) return 0;
    return work_layout(T, I, O, mid_dtype).total;
}

int qm_linear_forward(const void* x, int x_dtype, const void* w, int w_dtype, int64_t T, int64_t I, int64_t O, int hd_x,
                      const uint32_t* signs_x, int hd_w, const uint32_t* signs_w, void* packed_x, size_t packed_x_bytes,
                      void* packed_w, size_t packed_w_bytes, int packed_flags, void* y, int y_dtype, int codes_layout,
                      void* stream) {
    if (T < 0 || I < 0 || O < 0) return fail(QM_ERR_INVALID, "qm_linear_forward: negative extent");
    if (T == 0 || O == 0 || I == 0) return 0;
    if (I % 32) return fail(QM_ERR_INVALID, "qm_linear_forward: in_features %lld not a multiple of 32", (long long)I);
    const PackedLayout lx = packed_layout(T, I), lw = packed_layout(O, I);
    if (!packed_x || packed_x_bytes < lx.total || !aligned(packed_x, 256) || !packed_w || packed_w_bytes < lw.total ||
        !aligned(packed_w, 256))
        return fail(QM_ERR_INVALID, "qm_linear_forward: packed operand buffers need %zu and %zu bytes, 256-byte aligned", lx.total,
                    lw.total);
    uint8_t* px = static_cast<uint8_t*>(packed_x);
    uint8_t* pw = static_cast<uint8_t*>(packed_w);
    if (packed_flags & ~(QM_W_IS_PACKED | QM_X_IS_PACKED)) return fail(QM_ERR_INVALID, "qm_linear_forward: unknown packed_flags %d", packed_flags);
    const bool w_is_packed = packed_flags & QM_W_IS_PACKED, x_is_packed = packed_flags & QM_X_IS_PACKED;
    int rc = 0;
    if (!w_is_packed && !x_is_packed && pair_launches(codes_layout, T, I, O, hd_x, hd_w, 32) && x && w && y && valid_dtype(x_dtype) &&
        valid_dtype(w_dtype) && aligned(x, 16) && aligned(w, 16)) {
        // both forward quantizers in one grid
        const qm::RowmajorArgs ax{x, x_dtype, T, I, signs_x ? signs_x[0] : 0u, px + lx.c, px + lx.s, px + lx.m};
        const qm::RowmajorArgs aw{w, w_dtype, O, I, signs_w ? signs_w[0] : 0u, pw + lw.c, pw + lw.s, pw + lw.m};
        rc = from_hip(qm::quantize_rowmajor_hd32_tiled_pair(ax, aw, reinterpret_cast<hipStream_t>(stream)), "qm_linear_forward");
        if (rc) return rc;
    } else {
        if (!x_is_packed)
            rc = qm_quantize_mxfp4(x, x_dtype, T, I, hd_x, signs_x, QM_QUEST_RTN, 0, nullptr, 0, px + lx.c, px + lx.s, px + lx.m,
                                   nullptr, codes_layout, stream);
        if (rc) return rc;
        if (!w_is_packed) {
            rc = qm_quantize_mxfp4(w, w_dtype, O, I, hd_w, signs_w, QM_QUEST_RTN, 0, nullptr, 0, pw + lw.c, pw + lw.s, pw + lw.m,
                                   nullptr, codes_layout, stream);
            if (rc) return rc;
        }
    }
    return qm_gemm_mxfp4_tn(px + lx.c, px + lx.s, pw + lw.c, pw + lw.s, T, O, I, 1.0f, y, y_dtype, codes_layout, codes_layout, nullptr,
                            0, stream);
}

int qm_linear_backward(const void* e, int e_dtype, int64_t T, int64_t I, int64_t O, const void* packed_x, const void* packed_w,
                       int hd_x, const uint32_t* signs_x, int hd_w, const uint32_t* signs_w, int hd_g, const uint32_t* signs_g,
                       int g_mode, const uint64_t* seeds, int x_val_dtype, int w_val_dtype, int mid_dtype, int x_scale_dtype,
                       int w_scale_dtype, void* workspace, size_t workspace_bytes, void* gx, void* gw, int gw_dtype,
                       int codes_layout, int rotated_flags, const float* g_matrix, void* stream) {
    return qm_linear_backward_seeded(e, e_dtype, T, I, O, packed_x, packed_w, hd_x, signs_x, hd_w, signs_w, hd_g, signs_g, g_mode, seeds,
                                     x_val_dtype, w_val_dtype, mid_dtype, x_scale_dtype, w_scale_dtype, workspace, workspace_bytes, gx,
                                     gw, gw_dtype, codes_layout, rotated_flags, g_matrix, nullptr, stream);
}

int qm_linear_backward_seeded(const void* e, int e_dtype, int64_t T, int64_t I, int64_t O, const void* packed_x,
                              const void* packed_w, int hd_x, const uint32_t* signs_x, int hd_w, const uint32_t* signs_w, int hd_g,
                              const uint32_t* signs_g, int g_mode, const uint64_t* seeds, int x_val_dtype, int w_val_dtype,
                              int mid_dtype, int x_scale_dtype, int w_scale_dtype, void* workspace, size_t workspace_bytes, void* gx,
                              void* gw, int gw_dtype, int codes_layout, int rotated_flags, const float* g_matrix,
                              const uint64_t* seed_base, void* stream) {
    if (T < 0 || I < 0 || O < 0) return fail(QM_ERR_INVALID, "qm_linear_backward: negative extent");
    if (seed_base && (!aligned(seed_base, 8) || g_matrix || !pair_launches(codes_layout, T, I, O, hd_x, hd_w, hd_g)))
        return fail(QM_ERR_INVALID, "qm_linear_backward_seeded: a device seed base needs the tiled layout with Hadamard blocks 32, "
                                    "T, I, O multiples of 128, no dense rotation, and an 8-byte aligned pointer");
    if (T == 0 || O == 0 || I == 0) return 0;
    if (g_mode != QM_ABSMAX_RTN && g_mode != QM_ABSMAX_SR)
        return fail(QM_ERR_INVALID, "qm_linear_backward: gradient mode must be QM_ABSMAX_RTN or QM_ABSMAX_SR");
    if (!valid_dtype(mid_dtype)) return fail(QM_ERR_INVALID, "qm_linear_backward: mid_dtype %d", mid_dtype);
    if (gw_dtype != mid_dtype && !(mid_dtype == QM_BF16 && gw_dtype == QM_F32))
        return fail(QM_ERR_INVALID, "qm_linear_backward: gw_dtype must be mid_dtype, or QM_F32 with a bf16 mid_dtype (got %d, mid %d)",
                    gw_dtype, mid_dtype);
    if (I % 32 || O % 32 || T % 32)
        return fail(QM_ERR_INVALID, "qm_linear_backward: tokens, in_features and out_features must be multiples of 32 (T=%lld I=%lld O=%lld)",
                    (long long)T, (long long)I, (long long)O);
    if (!seeds || !packed_x || !aligned(packed_x, 256) || !packed_w || !aligned(packed_w, 256))
        return fail(QM_ERR_INVALID, "qm_linear_backward: null seeds or packed operand buffers");
    const PackedLayout lx = packed_layout(T, I), lw = packed_layout(O, I);
    const WorkLayout wl = work_layout(T, I, O, mid_dtype);
    if (!workspace || workspace_bytes < wl.total || !aligned(workspace, 256))
        return fail(QM_ERR_INVALID, "qm_linear_backward: workspace needs %zu bytes, 256-byte aligned", wl.total);
    const uint8_t* px = static_cast<const uint8_t*>(packed_x);
    const uint8_t* pw = static_cast<const uint8_t*>(packed_w);
    uint8_t* k = static_cast<uint8_t*>(workspace);
    // value = code * 2^k * fl32(4/3) on both operands of the two gradient products
    const float d = (float)(1.0 / 0.75);
    const float alpha = d * d;
    void* gws = wl.gemm_ws_bytes ? k + wl.gemm_ws : nullptr;
    hipStream_t hs = reinterpret_cast<hipStream_t>(stream);
    int rc;
    // rotated_flags: bit 0 (QM_GX_ROTATED): the caller undoes the activation quantizer's rotation itself (fused into its
    // next kernel, or a dense rotation it applies with a library product); the first product then lands in gx directly.
    // Bit 1 (QM_GW_ROTATED): the same for the weight quantizer's rotation and gw.
    if (rotated_flags & ~(QM_GX_ROTATED | QM_GW_ROTATED)) return fail(QM_ERR_INVALID, "qm_linear_backward: unknown rotated flags %d", rotated_flags);
    const bool gx_rotated = rotated_flags & QM_GX_ROTATED, gw_rotated = rotated_flags & QM_GW_ROTATED;
    if (gw_rotated && gw_dtype != mid_dtype) return fail(QM_ERR_INVALID, "qm_linear_backward: QM_GW_ROTATED needs gw_dtype == mid_dtype");
    void* gx_product = gx_rotated ? gx : static_cast<void*>(k + wl.gxq);
    void* gw_product = gw_rotated ? gw : static_cast<void*>(k + wl.gwq);
    // B8: gw in gw_dtype; a bf16 result widened to fp32 keeps its bf16 rounding (what converting it afterwards would give)
    const auto rotate_gw = [&]() -> int {
        if (gw_rotated) return 0;
        if (gw_dtype == mid_dtype)
            return qm_masked_hadamard_bwd(k + wl.gwq, mid_dtype, O, I, hd_w, w_scale_dtype, signs_w, pw + lw.m, gw, mid_dtype, stream);
        if (!valid_hd(hd_w) || I % hd_w || !gw || !aligned(gw, 16) || !valid_dtype(w_scale_dtype))
            return fail(QM_ERR_INVALID, "qm_linear_backward: bad hd_w, w_scale_dtype or gw");
        return from_hip(qm::masked_hadamard_bwd(k + wl.gwq, mid_dtype, O, I, hd_w, w_scale_dtype, make_signs(signs_w, hd_w), pw + lw.m, gw,
                                                gw_dtype, true, hs), "qm_linear_backward");
    };
    if (gx_rotated && hd_x != 32) return fail(QM_ERR_INVALID, "qm_linear_backward: gx_rotated needs hd_x == 32");
    // B3 + B7 and B6 + B8: where a gradient product runs on the persistent kernel's bf16 epilogue, the masked inverse
    // rotation of the forward quantizer is applied to the tile before it is stored and the product lands in gx / gw
    // directly (`fused` reports it); otherwise the product goes to the workspace and the rotation is a kernel of its own.
    const auto grad_product = [&](const uint8_t* ac, const uint8_t* as, const uint8_t* bc, const uint8_t* bs, int64_t M, int64_t N,
                                  int64_t K, void* plain_dst, void* final_dst, bool want_rotation, int hd, int final_dtype,
                                  const uint8_t* mask, const uint32_t* signs, int scale_dtype, bool& fused) -> int {
        fused = want_rotation && hd == 32 && final_dst && aligned(final_dst, 16) && valid_dtype(scale_dtype) && mask &&
                qm::gemm_will_rotate(as, bs, M, N, K, mid_dtype, final_dtype, gws, wl.gemm_ws_bytes);
        if (!fused)
            return qm_gemm_mxfp4_tn(ac, as, bc, bs, M, N, K, alpha, plain_dst, mid_dtype, codes_layout, codes_layout, gws, wl.gemm_ws_bytes, stream);
        bool done = false;
        const int r = from_hip(qm::gemm_mxfp4_tn_rotated(ac, as, bc, bs, M, N, K, alpha, final_dst, mid_dtype, codes_layout, codes_layout, gws,
                                                         wl.gemm_ws_bytes, mask, signs ? signs[0] : 0u, scale_dtype, final_dtype, &done, hs),
                               "qm_linear_backward");
        if (r) return r;
        return done ? 0 : fail(QM_ERR_INVALID, "qm_linear_backward: a gradient product did not run as planned");
    };
    bool gx_fused = false, gw_fused = false;
    const auto product_gx = [&]() {
        return grad_product(k + wl.ec, k + wl.es, k + wl.wtc, k + wl.wts, T, I, O, gx_product, gx, !gx_rotated, hd_x, mid_dtype, px + lx.m,
                            signs_x, x_scale_dtype, gx_fused);
    };
    const auto product_gw = [&]() {
        return grad_product(k + wl.etc, k + wl.ets, k + wl.xtc, k + wl.xts, O, I, T, gw_product, gw, !gw_rotated, hd_w, gw_dtype, pw + lw.m,
                            signs_w, w_scale_dtype, gw_fused);
    };
    if (g_matrix) {
        // a dense rotation in the gradient quantizer (rerotate="O32"): the same eight steps on the dense-rotation kernels
        if (hd_g != 32 || T % 128 || I % 128 || O % 128)
            return fail(QM_ERR_INVALID, "qm_linear_backward: a dense gradient rotation needs hd_g == 32 and T, I, O multiples of 128 "
                                        "(T=%lld I=%lld O=%lld)", (long long)T, (long long)I, (long long)O);
        rc = qm_quantize_mxfp4_dense(e, e_dtype, T, O, g_matrix, g_mode, 0, seeds[0], k + wl.ec, k + wl.es, nullptr, nullptr, codes_layout, stream);
        if (rc) return rc;
        rc = qm_requantize_transposed_mxfp4_dense(pw + lw.c, pw + lw.s, O, I, 1.0f, w_val_dtype, g_matrix, g_mode, seeds[1], k + wl.wtc,
                                                  k + wl.wts, nullptr, codes_layout, codes_layout, stream);
        if (rc) return rc;
        rc = product_gx();
        if (rc) return rc;
        rc = qm_quantize_mxfp4_dense(e, e_dtype, O, T, g_matrix, g_mode, 1, seeds[2], k + wl.etc, k + wl.ets, nullptr, nullptr, codes_layout, stream);
        if (rc) return rc;
        rc = qm_requantize_transposed_mxfp4_dense(px + lx.c, px + lx.s, T, I, 1.0f, x_val_dtype, g_matrix, g_mode, seeds[3], k + wl.xtc,
                                                  k + wl.xts, nullptr, codes_layout, codes_layout, stream);
        if (rc) return rc;
        rc = product_gw();
        if (rc) return rc;
        if (!gx_rotated && !gx_fused) {
            rc = qm_masked_hadamard_bwd(k + wl.gxq, mid_dtype, T, I, hd_x, x_scale_dtype, signs_x, px + lx.m, gx, mid_dtype, stream);
            if (rc) return rc;
        }
        return gw_fused ? 0 : rotate_gw();
    }
    if (pair_launches(codes_layout, T, I, O, hd_x, hd_w, hd_g) && e && gx && gw && valid_dtype(e_dtype) && aligned(e, 16) &&
        aligned(gx, 16) && aligned(gw, 16) && valid_dtype(x_val_dtype) && valid_dtype(w_val_dtype) &&
        valid_dtype(x_scale_dtype) && valid_dtype(w_scale_dtype)) {
        // seven launches: Q(e) with Q(e^T), Q(Q(W)^T) with Q(Q(x)^T), the two products, the two inverse rotations
        const uint32_t sg = signs_g ? signs_g[0] : 0u;
        rc = from_hip(qm::quantize_both_orientations_hd32_tiled(e, e_dtype, T, O, sg, g_mode, seeds[0], seeds[2], k + wl.ec, k + wl.es,
                                                                k + wl.etc, k + wl.ets, seed_base, hs), "qm_linear_backward");
        if (rc) return rc;
        const qm::RequantArgs rw{pw + lw.c, pw + lw.s, O, I, w_val_dtype, seeds[1], k + wl.wtc, k + wl.wts};
        const qm::RequantArgs rx{px + lx.c, px + lx.s, T, I, x_val_dtype, seeds[3], k + wl.xtc, k + wl.xts};
        rc = from_hip(qm::requantize_transposed_hd32_tiled_pair(rx, rw, sg, g_mode, seed_base, hs), "qm_linear_backward");
        if (rc) return rc;
        rc = product_gx();
        if (rc) return rc;
        rc = product_gw();
        if (rc) return rc;
        const bool need_x = !gx_rotated && !gx_fused, need_w = !gw_rotated && !gw_fused;
        if (!need_x) return need_w ? rotate_gw() : 0;
        if (!need_w)
            return qm_masked_hadamard_bwd(k + wl.gxq, mid_dtype, T, I, hd_x, x_scale_dtype, signs_x, px + lx.m, gx, mid_dtype, stream);
        return from_hip(qm::masked_hadamard_bwd_hd32_pair(k + wl.gxq, T * I, x_scale_dtype,
                                                          signs_x ? signs_x[0] : 0u, px + lx.m, gx, k + wl.gwq, O * I,
                                                          w_scale_dtype, signs_w ? signs_w[0] : 0u,
                                                          pw + lw.m, gw, mid_dtype, gw_dtype, hs), "qm_linear_backward");
    }
    if (seed_base) return fail(QM_ERR_INVALID, "qm_linear_backward_seeded: null, misaligned or ill-typed tensors");
    rc = qm_quantize_mxfp4(e, e_dtype, T, O, hd_g, signs_g, g_mode, 0, nullptr, seeds[0], k + wl.ec, k + wl.es, nullptr, nullptr,
                           codes_layout, stream);
    if (rc) return rc;
    rc = qm_requantize_transposed_mxfp4(pw + lw.c, pw + lw.s, O, I, 1.0f, w_val_dtype, hd_g, signs_g, g_mode, nullptr, seeds[1],
                                        k + wl.wtc, k + wl.wts, nullptr, codes_layout, codes_layout, stream);
    if (rc) return rc;
    rc = product_gx();
    if (rc) return rc;
    rc = qm_quantize_mxfp4(e, e_dtype, O, T, hd_g, signs_g, g_mode, 1, nullptr, seeds[2], k + wl.etc, k + wl.ets, nullptr, nullptr,
                           codes_layout, stream);
    if (rc) return rc;
    rc = qm_requantize_transposed_mxfp4(px + lx.c, px + lx.s, T, I, 1.0f, x_val_dtype, hd_g, signs_g, g_mode, nullptr, seeds[3],
                                        k + wl.xtc, k + wl.xts, nullptr, codes_layout, codes_layout, stream);
    if (rc) return rc;
    rc = product_gw();
    if (rc) return rc;
    if (!gx_rotated && !gx_fused) {
        rc = qm_masked_hadamard_bwd(k + wl.gxq, mid_dtype, T, I, hd_x, x_scale_dtype, signs_x, px + lx.m, gx, mid_dtype, stream);
        if (rc) return rc;
    }
    return gw_fused ? 0 : rotate_gw();
}

int qm_rmsnorm_quantize_mxfp4(const void* x, int x_dtype, const void* add, int add_dtype, void* x_sum, const float* gain, float eps,
                              int64_t rows, int64_t cols, const uint32_t* sign_bits, void* packed, size_t packed_bytes,
                              float* factor, int codes_layout, void* stream) {
    if (!valid_layout(codes_layout)) return fail(QM_ERR_INVALID, "qm_rmsnorm_quantize_mxfp4: unknown codes_layout %d", codes_layout);
    if (!valid_dtype(x_dtype)) return fail(QM_ERR_INVALID, "qm_rmsnorm_quantize_mxfp4: x_dtype %d is not QM_BF16/QM_F32", x_dtype);
    if (rows < 0 || cols <= 0 || cols % 32)
        return fail(QM_ERR_INVALID, "qm_rmsnorm_quantize_mxfp4: need rows >= 0 and cols a positive multiple of 32 (got [%lld, %lld])",
                    (long long)rows, (long long)cols);
    if (rows == 0) return 0;
    if (codes_layout == QM_LAYOUT_TILED && (rows % 16 || cols % 128))
        return fail(QM_ERR_INVALID, "qm_rmsnorm_quantize_mxfp4: tiled codes need rows %% 16 == 0 and cols %% 128 == 0 (rows=%lld cols=%lld)",
                    (long long)rows, (long long)cols);
    const PackedLayout l = packed_layout(rows, cols);
    if (!x || !gain || !factor || !packed || packed_bytes < l.total)
        return fail(QM_ERR_INVALID, "qm_rmsnorm_quantize_mxfp4: x, gain, factor must be non-null and packed hold %zu bytes", l.total);
    if (!aligned(x, 16) || !aligned(gain, 16) || !aligned(packed, 256) || !aligned(factor, 4) || !aligned(add, 16) || !aligned(x_sum, 16))
        return fail(QM_ERR_UNALIGNED, "qm_rmsnorm_quantize_mxfp4: x, add, x_sum and gain need 16-byte, packed 256-byte alignment");
    if (add && (x_dtype != QM_F32 || !valid_dtype(add_dtype) || !x_sum))
        return fail(QM_ERR_INVALID, "qm_rmsnorm_quantize_mxfp4: a residual summand needs an fp32 x, a valid add_dtype and x_sum");
    uint8_t* p = static_cast<uint8_t*>(packed);
    return from_hip(qm::rmsnorm_quantize_hd32(x, x_dtype, add, add_dtype, x_sum, gain, eps, rows, cols, sign_bits ? sign_bits[0] : 0u, p + l.c, p + l.s,
                                              p + l.m, factor, codes_layout == QM_LAYOUT_TILED, reinterpret_cast<hipStream_t>(stream)),
                    "qm_rmsnorm_quantize_mxfp4");
}

int qm_swiglu_quantize_mxfp4(const void* h12, int dtype, int64_t rows, int64_t hidden, const uint32_t* sign_bits, void* packed,
                             size_t packed_bytes, int codes_layout, void* stream) {
    if (!valid_layout(codes_layout)) return fail(QM_ERR_INVALID, "qm_swiglu_quantize_mxfp4: unknown codes_layout %d", codes_layout);
    if (!valid_dtype(dtype)) return fail(QM_ERR_INVALID, "qm_swiglu_quantize_mxfp4: dtype %d is not QM_BF16/QM_F32", dtype);
    if (rows < 0 || hidden <= 0 || hidden % 32)
        return fail(QM_ERR_INVALID, "qm_swiglu_quantize_mxfp4: need rows >= 0 and hidden a positive multiple of 32 (got [%lld, %lld])",
                    (long long)rows, (long long)hidden);
    if (rows == 0) return 0;
    if (codes_layout == QM_LAYOUT_TILED && (rows % 16 || hidden % 128))
        return fail(QM_ERR_INVALID, "qm_swiglu_quantize_mxfp4: tiled codes need rows %% 16 == 0 and hidden %% 128 == 0 (rows=%lld hidden=%lld)",
                    (long long)rows, (long long)hidden);
    const PackedLayout l = packed_layout(rows, hidden);
    if (!h12 || !packed || packed_bytes < l.total)
        return fail(QM_ERR_INVALID, "qm_swiglu_quantize_mxfp4: h12 must be non-null and packed hold %zu bytes", l.total);
    if (!aligned(h12, 16) || !aligned(packed, 256))
        return fail(QM_ERR_UNALIGNED, "qm_swiglu_quantize_mxfp4: h12 needs 16-byte, packed 256-byte alignment");
    uint8_t* p = static_cast<uint8_t*>(packed);
    return from_hip(qm::swiglu_quantize_hd32(h12, dtype, rows, hidden, sign_bits ? sign_bits[0] : 0u, p + l.c, p + l.s, p + l.m,
                                             codes_layout == QM_LAYOUT_TILED, reinterpret_cast<hipStream_t>(stream)),
                    "qm_swiglu_quantize_mxfp4");
}

size_t qm_rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols) {
    if (rows < 0 || cols <= 0 || cols % 32 || cols > 8192) return 0;
    return up256(qm::rmsnorm_backward_workspace_bytes(rows, cols));
}

int qm_rmsnorm_backward(const void* gy, int gy_dtype, const void* x, int x_dtype, const float* gain, const float* factor,
                        int64_t rows, int64_t cols, const uint8_t* maskbits, const uint32_t* sign_bits, int scale_dtype,
                        const void* skip, void* dx, void* dx_bf16, float* dgain, void* workspace, size_t workspace_bytes,
                        void* stream) {
    if (!valid_dtype(gy_dtype) || !valid_dtype(x_dtype) || (maskbits && !valid_dtype(scale_dtype)))
        return fail(QM_ERR_INVALID, "qm_rmsnorm_backward: dtypes must be QM_BF16/QM_F32");
    if (rows < 0 || cols <= 0 || cols % 32 || cols > 8192)
        return fail(QM_ERR_INVALID, "qm_rmsnorm_backward: need rows >= 0 and cols a multiple of 32 in [32, 8192] (got [%lld, %lld])",
                    (long long)rows, (long long)cols);
    if (!dgain) return fail(QM_ERR_INVALID, "qm_rmsnorm_backward: dgain must be non-null");
    if (rows > 0 && (!gy || !x || !gain || !factor || !dx || !workspace || workspace_bytes < qm::rmsnorm_backward_workspace_bytes(rows, cols)))
        return fail(QM_ERR_INVALID, "qm_rmsnorm_backward: null tensor, or workspace below %zu bytes", qm_rmsnorm_backward_workspace_bytes(rows, cols));
    if (!aligned(maskbits, 4)) return fail(QM_ERR_UNALIGNED, "qm_rmsnorm_backward: maskbits needs 4-byte alignment");
    if (!aligned(skip, 16) || !aligned(dx_bf16, 8) || !aligned(gy, 8) || !aligned(x, 8) || !aligned(dx, 8) || !aligned(gain, 16) || !aligned(workspace, 16) ||
        (gy_dtype == QM_F32 && !aligned(gy, 16)) || (x_dtype == QM_F32 && (!aligned(x, 16) || !aligned(dx, 16))))
        return fail(QM_ERR_UNALIGNED, "qm_rmsnorm_backward: tensors need 16-byte alignment");
    return from_hip(qm::rmsnorm_backward(gy, gy_dtype, x, x_dtype, gain, factor, rows, cols, maskbits, sign_bits ? sign_bits[0] : 0u,
                                         maskbits ? scale_dtype : QM_F32, skip, dx, dx_bf16, dgain, workspace,
                                         reinterpret_cast<hipStream_t>(stream)),
                    "qm_rmsnorm_backward");
}

int qm_swiglu_backward(const void* g, int g_dtype, const void* h12, int dtype, int64_t rows, int64_t hidden,
                       const uint8_t* maskbits, const uint32_t* sign_bits, int scale_dtype, void* d_h12, void* stream) {
    if (!valid_dtype(g_dtype) || !valid_dtype(dtype) || (maskbits && !valid_dtype(scale_dtype)))
        return fail(QM_ERR_INVALID, "qm_swiglu_backward: dtypes must be QM_BF16/QM_F32");
    if (rows < 0 || hidden <= 0 || hidden % 4 || (maskbits && hidden % 32))
        return fail(QM_ERR_INVALID, "qm_swiglu_backward: need rows >= 0 and hidden a positive multiple of 4 (of 32 with mask bits) "
                                    "(got [%lld, %lld])", (long long)rows, (long long)hidden);
    if (rows == 0) return 0;
    if (!g || !h12 || !d_h12) return fail(QM_ERR_INVALID, "qm_swiglu_backward: g, h12 and d_h12 must be non-null");
    if (!aligned(g, 16) || !aligned(h12, 16) || !aligned(d_h12, 16))
        return fail(QM_ERR_UNALIGNED, "qm_swiglu_backward: tensors need 16-byte alignment");
    return from_hip(qm::swiglu_backward(g, g_dtype, h12, dtype, rows, hidden, maskbits, sign_bits ? sign_bits[0] : 0u,
                                        maskbits ? scale_dtype : QM_F32, d_h12, reinterpret_cast<hipStream_t>(stream)),
                    "qm_swiglu_backward");
}

namespace {
int check_rope(const char* who, int dtype_a, int dtype_b, int64_t rows, int64_t seq_len, int64_t n_embd, int head_dim) {
    if (!valid_dtype(dtype_a) || !valid_dtype(dtype_b)) return fail(QM_ERR_INVALID, "%s: dtypes must be QM_BF16/QM_F32", who);
    if (rows < 0 || seq_len <= 0 || n_embd <= 0 || head_dim <= 0 || head_dim % 8 || n_embd % head_dim || n_embd > (1 << 24) ||
        seq_len > (1 << 30))
        return fail(QM_ERR_INVALID, "%s: need rows >= 0, seq_len > 0, head_dim a positive multiple of 8 and n_embd a multiple of "
                                    "head_dim (rows=%lld seq_len=%lld n_embd=%lld head_dim=%d)",
                    who, (long long)rows, (long long)seq_len, (long long)n_embd, head_dim);
    return 0;
}
}  // namespace

int qm_rope_split_qkv(const void* qkv, int qkv_dtype, int64_t rows, int64_t seq_len, int64_t n_embd, int head_dim,
                      const float* table, void* q, void* k, void* v, int out_dtype, void* stream) {
    if (int rc = check_rope("qm_rope_split_qkv", qkv_dtype, out_dtype, rows, seq_len, n_embd, head_dim)) return rc;
    if (rows == 0) return 0;
    if (!qkv || !table || !q || !k || !v) return fail(QM_ERR_INVALID, "qm_rope_split_qkv: qkv, table, q, k, v must be non-null");
    if (!aligned(qkv, 16) || !aligned(table, 16) || !aligned(q, 16) || !aligned(k, 16) || !aligned(v, 16))
        return fail(QM_ERR_UNALIGNED, "qm_rope_split_qkv: tensors need 16-byte alignment");
    return from_hip(qm::rope_split_qkv(qkv, qkv_dtype, rows, (int)seq_len, (int)n_embd, head_dim, table, q, k, v, out_dtype,
                                       reinterpret_cast<hipStream_t>(stream)),
                    "qm_rope_split_qkv");
}

int qm_rope_merge_qkv_grad(const void* dq, const void* dk, const void* dv, int grad_dtype, int64_t rows, int64_t seq_len,
                           int64_t n_embd, int head_dim, const float* table, void* d_qkv, int out_dtype, void* stream) {
    if (int rc = check_rope("qm_rope_merge_qkv_grad", grad_dtype, out_dtype, rows, seq_len, n_embd, head_dim)) return rc;
    if (rows == 0) return 0;
    if (!dq || !dk || !dv || !table || !d_qkv)
        return fail(QM_ERR_INVALID, "qm_rope_merge_qkv_grad: dq, dk, dv, table, d_qkv must be non-null");
    if (!aligned(dq, 16) || !aligned(dk, 16) || !aligned(dv, 16) || !aligned(table, 16) || !aligned(d_qkv, 16))
        return fail(QM_ERR_UNALIGNED, "qm_rope_merge_qkv_grad: tensors need 16-byte alignment");
    return from_hip(qm::rope_merge_qkv_grad(dq, dk, dv, grad_dtype, rows, (int)seq_len, (int)n_embd, head_dim, table, d_qkv, out_dtype,
                                            reinterpret_cast<hipStream_t>(stream)),
                    "qm_rope_merge_qkv_grad");
}

}  // extern "C"
