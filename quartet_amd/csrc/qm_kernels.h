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

// Code-byte layouts of a packed [R, C] tensor.  ROWMAJOR: [R][C/2].  TILED (R % 16 == 0, C % 128 == 0):
// [R/16][C/128][16 rows][64 bytes] -- the 16 rows x 128 elements one GEMM wave-load fetches are 1 KiB contiguous.
enum CodeLayout : int { LAYOUT_ROWMAJOR = 0, LAYOUT_TILED = 1 };

// byte offset of the 64-byte piece (row r, column block kb) in the tiled layout
__host__ __device__ inline int64_t tiled_code_offset(int64_t r, int64_t kb, int64_t kblocks) {
    return (((r >> 4) * kblocks + kb) << 10) + ((r & 15) << 6);
}

hipError_t quantize_mxfp4(const void* x, int dtype, int64_t rows, int64_t cols, int hd, const SignBits& sb, int mode,
                          bool transposed_in, const float* u, uint64_t seed, uint8_t* codes, uint8_t* scales,
                          uint8_t* maskbits, void* dequant, int codes_layout, hipStream_t stream);
// whether quantize_mxfp4 / requantize_transposed_mxfp4 can emit (read) tiled codes for these arguments
bool quantize_supports_tiled(int64_t rows, int64_t cols, int hd, int mode, bool transposed_in, const float* u,
                             const uint8_t* maskbits);
bool requantize_supports_tiled(int64_t R, int64_t C, int hd, int mode, const float* u);
bool gemm_supports_tiled(int64_t M, int64_t N, int64_t K);

// hd = 32 fast path (one MX group per lane, hardware FP4 converts); row-major input, RTN or Philox SR
hipError_t quantize_rowmajor_hd32(const void* x, int dtype, int64_t rows, int64_t cols, uint32_t sign_word, int mode,
                                  uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                                  bool tiled, bool rotate, hipStream_t stream);

hipError_t quantize_rowmajor_wide(const void* x, int dtype, int64_t n, int hd, const SignBits& sb, int mode, uint64_t seed,
                                  uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant, hipStream_t stream);

hipError_t quantize_transposed_hd32(const void* x, int dtype, int64_t P, int64_t Q, uint32_t sign_word, int mode,
                                    uint64_t seed, uint8_t* codes, uint8_t* scales, void* dequant, bool tiled,
                                    hipStream_t stream);
hipError_t requantize_transposed_hd32(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C, float post,
                                      int val_dtype, uint32_t sign_word, int mode, uint64_t seed, uint8_t* codes,
                                      uint8_t* scales, void* dequant, bool tiled_in, bool tiled_out, hipStream_t stream);

// The same with a dense 32x32 rotation instead of the Hadamard block (matrix: device pointer, [32][32] fp32, H[k][j])
hipError_t quantize_rowmajor_dense(const void* x, int dtype, int64_t rows, int64_t cols, const float* matrix, int mode,
                                   uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                                   bool tiled, hipStream_t stream);
hipError_t quantize_transposed_dense(const void* x, int dtype, int64_t P, int64_t Q, const float* matrix, int mode,
                                     uint64_t seed, uint8_t* codes, uint8_t* scales, void* dequant, bool tiled,
                                     hipStream_t stream);
hipError_t requantize_transposed_dense(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C, float post,
                                       int val_dtype, const float* matrix, int mode, uint64_t seed, uint8_t* codes,
                                       uint8_t* scales, void* dequant, bool tiled_in, bool tiled_out, hipStream_t stream);
// shape-checked front ends of the three (what the C ABI calls); hipErrorInvalidValue for shapes they do not serve
hipError_t quantize_mxfp4_dense(const void* x, int dtype, int64_t rows, int64_t cols, const float* matrix, int mode,
                                bool transposed_in, uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits,
                                void* dequant, int codes_layout, hipStream_t stream);
hipError_t requantize_transposed_mxfp4_dense(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C,
                                             float post, int val_dtype, const float* matrix, int mode, uint64_t seed,
                                             uint8_t* codes_out, uint8_t* scales_out, void* dequant, int in_layout,
                                             int out_layout, hipStream_t stream);

// Pairs of independent quantizer launches issued as one grid (Hadamard block 32, tiled codes in and out).
struct RowmajorArgs {
    const void* x;
    int dtype;
    int64_t rows, cols;
    uint32_t sign_word;
    uint8_t* codes;
    uint8_t* scales;
    uint8_t* maskbits;
};
struct RequantArgs {
    const uint8_t* codes_in;
    const uint8_t* scales_in;
    int64_t R, C;
    int val_dtype;
    uint64_t seed;
    uint8_t* codes;
    uint8_t* scales;
};
hipError_t quantize_rowmajor_hd32_tiled_pair(const RowmajorArgs& a, const RowmajorArgs& b, hipStream_t stream);
hipError_t quantize_both_orientations_hd32_tiled(const void* e, int dtype, int64_t T, int64_t O, uint32_t sign_word, int mode,
                                                 uint64_t seed_rows, uint64_t seed_transposed, uint8_t* codes_rows,
                                                 uint8_t* scales_rows, uint8_t* codes_transposed, uint8_t* scales_transposed,
                                                 const uint64_t* seed_base, hipStream_t stream);
// seed_base: null, or device memory holding a value the kernels add to every seed when they run
hipError_t requantize_transposed_hd32_tiled_pair(const RequantArgs& a, const RequantArgs& b, uint32_t sign_word, int mode,
                                                 const uint64_t* seed_base, hipStream_t stream);
hipError_t masked_hadamard_bwd_hd32_pair(const void* ga, int64_t na, int scale_dtype_a, uint32_t sign_a, const uint8_t* mask_a, void* out_a,
                                         const void* gb, int64_t nb, int scale_dtype_b, uint32_t sign_b, const uint8_t* mask_b, void* out_b,
                                         int dtype, int out_dtype_b, hipStream_t stream);

// Producers fused into the forward quantizer (Hadamard block 32, quest RTN, clip mask) and their backward passes
hipError_t rmsnorm_quantize_hd32(const void* x, int dtype, const void* add, int add_dtype, void* xsum, const float* gain, float eps,
                                 int64_t rows, int64_t cols, uint32_t sign_word, uint8_t* codes, uint8_t* scales, uint8_t* maskbits,
                                 float* factor, bool tiled, hipStream_t stream);
hipError_t swiglu_quantize_hd32(const void* h12, int dtype, int64_t rows, int64_t hidden, uint32_t sign_word,
                                uint8_t* codes, uint8_t* scales, uint8_t* maskbits, bool tiled, hipStream_t stream);
size_t rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols);
hipError_t rmsnorm_backward(const void* gy, int gy_dtype, const void* x, int x_dtype, const float* gain,
                            const float* factor, int64_t rows, int64_t cols, const uint8_t* maskbits, uint32_t sign_word,
                            int scale_dtype, const void* skip, void* dx, void* dx_bf16, float* dgain, void* workspace,
                            hipStream_t stream);
hipError_t swiglu_backward(const void* g, int g_dtype, const void* h12, int dtype, int64_t rows, int64_t hidden,
                           const uint8_t* maskbits, uint32_t sign_word, int scale_dtype, void* d_h12, hipStream_t stream);

// Rotary embedding of the fused attention projection: split + rotate, and the merge + inverse rotation of its backward
hipError_t rope_split_qkv(const void* qkv, int qkv_dtype, int64_t rows, int seq_len, int C, int head_dim, const float* table,
                          void* q, void* k, void* v, int out_dtype, hipStream_t stream);
hipError_t rope_merge_qkv_grad(const void* dq, const void* dk, const void* dv, int grad_dtype, int64_t rows, int seq_len, int C,
                               int head_dim, const float* table, void* d_qkv, int out_dtype, hipStream_t stream);

hipError_t requantize_transposed_mxfp4(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C,
                                       float post, int val_dtype, int hd, const SignBits& sb, int mode, const float* u,
                                       uint64_t seed, uint8_t* codes_out, uint8_t* scales_out, void* dequant,
                                       int in_layout, int out_layout, hipStream_t stream);

hipError_t gemm_mxfp4_tn(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                         const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype,
                         int a_layout, int b_layout, void* workspace, size_t workspace_bytes, hipStream_t stream);
// the same product with the masked inverse Hadamard rotation of the layer's backward pass (hd 32, along N) fused into the
// store of the result where the kernel serving the shape can do it: in the persistent kernel's bf16 epilogue (c_dtype and
// rot_out_dtype both BF16), or in the ordered reduction of a product cut into K ranges (the product rounded to c_dtype,
// the rotated result stored in rot_out_dtype: c_dtype, or F32 holding the bf16-rounded result).  *rotated reports whether
// it was; c then holds rot_out_dtype elements, otherwise the plain product in c_dtype.
bool gemm_will_rotate(const uint8_t* a_scales, const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, int c_dtype, int rot_out_dtype,
                      const void* workspace, size_t workspace_bytes);
hipError_t gemm_mxfp4_tn_rotated(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                                 const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype,
                                 int a_layout, int b_layout, void* workspace, size_t workspace_bytes, const uint8_t* rot_mask,
                                 uint32_t rot_signs, int rot_scale_dtype, int rot_out_dtype, bool* rotated, hipStream_t stream);
// the reduction of a product cut into K ranges with that rotation applied to the reduced values (hadamard_bwd.hip)
hipError_t splitk_reduce_rotated(const float* partial, int splits, int64_t mn, float alpha, int mid_dtype, const uint8_t* maskbits,
                                 uint32_t sign_word, int scale_dtype, void* out, int out_dtype, hipStream_t stream);
size_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
// C = alpha * A (packed MXFP4 [M, K]) x B (bf16 [K, N] row-major): K % 64 == 0, N % 8 == 0
bool gemm_fp4_bf16_nn_supported(int64_t M, int64_t N, int64_t K);
hipError_t gemm_fp4_bf16_nn(const uint8_t* a_codes, const uint8_t* a_scales, const void* b, int64_t M, int64_t N, int64_t K,
                            float alpha, void* c, int c_dtype, hipStream_t stream);
// measurement aid: one launch of the persistent kernel that records the shader clock around every tile's K loop and epilogue
int gemm_phase_stamps_per_group();
hipError_t gemm_tile_phases(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                            int64_t M, int64_t N, int64_t K, float alpha, void* c, int a_layout, int b_layout,
                            const uint8_t* rot_mask, unsigned long long* stamps, size_t stamps_bytes, int* grid_out, hipStream_t stream);
// measurement aid: the FP4 matrix instruction alone (see gemm.hip)
int mfma_only_blocks();
hipError_t mfma_only(const uint8_t* operands, float* sink, int iters, hipStream_t stream);

hipError_t masked_hadamard_bwd(const void* g, int g_dtype, int64_t rows, int64_t cols, int hd, int scale_dtype,
                               const SignBits& sb, const uint8_t* maskbits, void* out, int out_dtype,
                               bool round_to_g_dtype, hipStream_t stream);

hipError_t dequantize_mxfp4(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C, float post, void* out,
                            int out_dtype, hipStream_t stream);

}  // namespace qm
