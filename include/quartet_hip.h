/*
 * quartet_hip.h -- C ABI of libquartet_hip.so: the MI355X (gfx950) kernels behind Quartet's
 * MXFP4 quantized-linear path.
 *
 * Conventions
 *   - every tensor pointer is a DEVICE pointer owned by the caller; outputs are pre-allocated;
 *   - `stream` is a hipStream_t (NULL = default stream); calls are asynchronous on it;
 *   - return value: 0 = ok, < 0 = rejected arguments (nothing was launched; qm_last_error()
 *     holds the reason, thread-local), > 0 = a hipError_t from the launch;
 *   - packed MXFP4 tensor of logical shape [R, C] (C % 32 == 0):
 *       codes  uint8 [R, C/2]   E2M1, element 2i in the low nibble of byte i, sign in bit 3
 *                               (QM_LAYOUT_ROWMAJOR); or, for R % 16 == 0 and C % 128 == 0, QM_LAYOUT_TILED:
 *                               the same bytes as [R/16][C/128][16 rows][64 bytes], so that the 16 rows x 128
 *                               elements one GEMM wave-load fetches are 1 KiB contiguous.  Scales and mask bits
 *                               are row-major in both layouts.
 *       scales uint8 [R, C/32]  E8M0 (value 2^(byte-127)), one per 32 consecutive elements
 *       mask   uint8 [R, C/8]   bit i of byte j = clip mask of element 8j+i
 *   - `sign_bits`: HOST pointer to ceil(hd/32) uint32 words, bit j set = rotated column j is
 *     negated (the accumulated +-1 diagonal of re_randomize), or NULL for no sign flips.
 *
 * The reference has no FFI; each entry point below names the Python/Triton call it replaces
 * (paths relative to the reference checkout).
 */
#ifndef QUARTET_HIP_H
#define QUARTET_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { QM_BF16 = 0, QM_F32 = 1 };
/* scale rule + rounding: quest = std-based scale (QuestMXFP4Quantizer), absmax = max/(3/4)
 * (AlbertTsengQuantizer); RTN = ties toward zero, SR = stochastic rounding */
enum { QM_QUEST_RTN = 0, QM_ABSMAX_RTN = 1, QM_ABSMAX_SR = 2, QM_QUEST_SR = 3 };

/* layout of a packed tensor's code bytes (see above); producers and consumers must agree per tensor */
enum { QM_LAYOUT_ROWMAJOR = 0, QM_LAYOUT_TILED = 1 };
/* qm_linear_forward: which packed operand buffers already hold their operand on entry */
enum { QM_W_IS_PACKED = 1, QM_X_IS_PACKED = 2 };
/* rotated_flags of qm_linear_backward */
enum { QM_GX_ROTATED = 1, QM_GW_ROTATED = 2 };

#define QM_ERR_INVALID (-1)
#define QM_ERR_UNALIGNED (-2)

int qm_version(void);
/* message of the last failed call on this thread ("" if none) */
const char* qm_last_error(void);

/*
 * Fused block-Hadamard rotation + MXFP4 quantization of a logical [rows, cols] tensor along cols.
 * Replaces mxfp4_forward_kernel_wrapper (src/models/quantization/quantizers/mxfp4_triton.py:177-220)
 * as called by QuestMXFP4QuantizerFn.forward (quantizers/mxfp4.py:129-140, mode QM_QUEST_RTN with
 * maskbits) and AlbertTsengQuantizerFn.forward (quantizers/mxfp4.py:17-28, QM_ABSMAX_RTN/SR).
 *   x            input, dtype x_dtype; row-major [rows, cols], or, when transposed_in != 0,
 *                row-major [cols, rows] (the kernel quantizes its transpose: this is
 *                `e.T.contiguous()` + quantize of backward.py:81 in one pass)
 *   hadamard_dim 32, 64 or 128; cols % hadamard_dim == 0.  hadamard_dim 1 = the input is already rotated (the dense
 *                random rotation of rerotate="O32", mxfp4.py:61-64, applied by the caller): groups of 32 are
 *                quantized as they are; row-major input and codes only, sign_bits == NULL, u == NULL
 *   u            SR modes: device floats in [0,1) indexed by logical flat offset, or NULL to draw
 *                them in-kernel from Philox4x32-7 keyed by (seed, offset / 16): element j of a call takes the top
 *                22 bits of word j / 4 rotated left by 8 (j % 4) bits
 *   codes/scales outputs (required); maskbits, dequant optional (NULL to skip); dequant has
 *                x_dtype and logical shape and holds what the reference kernel returns
 *   codes_layout QM_LAYOUT_TILED needs hadamard_dim 32, rows % 16 == 0, cols % 128 == 0, u == NULL for
 *                the SR modes and, with transposed_in, maskbits == NULL; rejected otherwise
 */
int qm_quantize_mxfp4(const void* x, int x_dtype, int64_t rows, int64_t cols, int hadamard_dim,
                      const uint32_t* sign_bits, int mode, int transposed_in, const float* u,
                      uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits,
                      void* dequant, int codes_layout, void* stream);

/*
 * De-quantize a packed [R, C] tensor, transpose it, rotate and re-quantize along R:
 * outputs codes_out [C, R/2], scales_out [C, R/32].  Replaces
 * `g_quantizer(wq.T.contiguous())` / `g_quantizer(xq.T.contiguous())`
 * (src/models/quantization/backward.py:73,82) on the saved quantized operand, and the role of
 * backward_qt_bf16 in notebooks/benchmark_mxfp4.ipynb.
 *   post       1.0 if the input was quest-coded, fl32(4/3) if absmax-coded
 *   val_dtype  dtype the reference would hold the de-quantized tensor in (selects the rounding
 *              of the Hadamard constant and of the de-quantized values)
 *   in_layout / out_layout  layouts of codes_in / codes_out; QM_LAYOUT_TILED on either side needs
 *              hadamard_dim 32, R % 128 == 0, C % 128 == 0 and u == NULL for the SR modes
 */
int qm_requantize_transposed_mxfp4(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R,
                                   int64_t C, float post, int val_dtype, int hadamard_dim,
                                   const uint32_t* sign_bits, int mode, const float* u,
                                   uint64_t seed, uint8_t* codes_out, uint8_t* scales_out,
                                   void* dequant, int in_layout, int out_layout, void* stream);

/*
 * The two quantizers with a dense 32 x 32 rotation in place of the Hadamard block: the matrix a quantizer holds after
 * re_randomize with rerotate="O32" (U V^T of a Gaussian matrix's SVD, quantizers/mxfp4.py:61-64), which the reference
 * applies with tl.dot inside its kernel (mxfp4_triton.py:44-45).  Each group of 32 consecutive elements g becomes
 * g . matrix, evaluated on the matrix pipe as out[j] = fma(g[31], H[31][j], ... fma(g[0], H[0][j], 0)), then quantized
 * as by qm_quantize_mxfp4 / qm_requantize_transposed_mxfp4.
 *   matrix  DEVICE pointer to [32][32] fp32, row-major (H[k][j]); entries are rounded to x_dtype / val_dtype first,
 *           as the reference casts its matrix to the tensor's dtype (mxfp4.py:49)
 *   SR modes draw from the in-kernel Philox stream of `seed`.
 * qm_quantize_mxfp4_dense: cols % 32 == 0; transposed_in needs cols % 128 == 0, rows % 8 == 0 and maskbits == NULL;
 *   QM_LAYOUT_TILED needs rows % 16 == 0 and cols % 128 == 0.
 * qm_requantize_transposed_mxfp4_dense: R % 128 == 0, C % 32 == 0; QM_LAYOUT_TILED on either side needs C % 128 == 0.
 */
int qm_quantize_mxfp4_dense(const void* x, int x_dtype, int64_t rows, int64_t cols, const float* matrix, int mode,
                            int transposed_in, uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits,
                            void* dequant, int codes_layout, void* stream);
int qm_requantize_transposed_mxfp4_dense(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C,
                                         float post, int val_dtype, const float* matrix, int mode, uint64_t seed,
                                         uint8_t* codes_out, uint8_t* scales_out, void* dequant, int in_layout,
                                         int out_layout, void* stream);

/*
 * C[M, N] = alpha * A[M, K] . B[N, K]^T on packed MXFP4 operands, fp32 accumulation.
 * Replaces F.linear / einsum on de-quantized operands (src/models/quantization/backward.py:62,
 * 71-75, 79-83) and matmul_mxf4_bf16_tn of notebooks/benchmark_mxfp4.ipynb.  K % 32 == 0.
 * alpha carries the per-operand constants of absmax coding (fl32(4/3) each).
 * Alignment: a_codes and b_codes 16 bytes, scales 4 bytes; c 16 bytes for the shapes the tile kernels serve (M, N
 * multiples of 64 and >= 256, K % 128 == 0: they store c in 16-byte pieces), 4 bytes otherwise; QM_ERR_UNALIGNED
 * if not.
 * a_layout / b_layout: layouts of a_codes / b_codes; QM_LAYOUT_TILED needs M and N multiples of 64 and
 * at least 256, and K % 128 == 0 (the shapes the 256x256-tile kernels serve).
 * workspace: optional scratch (NULL, 0 for none).  With qm_gemm_workspace_bytes(M, N, K) > 0 bytes of it, 16-byte
 * aligned, a product with few output tiles and a long K is cut into K ranges whose fp32 partial sums are added in
 * a fixed order (results are reproducible, but differ in rounding from the unsplit product).
 */
size_t qm_gemm_workspace_bytes(int64_t M, int64_t N, int64_t K);
int qm_gemm_mxfp4_tn(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                     const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c,
                     int c_dtype, int a_layout, int b_layout, void* workspace, size_t workspace_bytes,
                     void* stream);

/*
 * c[M, N] = alpha * A @ B with A packed MXFP4 (row-major codes [M, K/2], E8M0 scales [M, K/32]) and B plain bf16
 * [K, N] row-major: the two gradient products of the scheme that quantizes only the error signal,
 * QEW_QEtXFn.backward (src/models/quantization/backward.py:31-43): grad_x = Q(e) @ w with A = Q(e) [T, O], B = w [O, I],
 * and grad_w = Q(e^T) @ x with A = Q(e^T) [O, T], B = x [T, I] -- the saved operands exactly as they lie in memory, no
 * transposed copy, no de-quantized tensor (the reference multiplies a de-quantized bf16 copy of Q(e) with a library GEMM).
 * Codes are decoded to bf16 in registers (exact), products accumulate in fp32.  alpha carries the quantizer's
 * post-scale (fl32(4/3) for the absmax modes).  c_dtype QM_BF16 or QM_F32.  A scale byte of 0 reads as zero (not
 * 2^-127).  Needs K % 64 == 0 and N % 8 == 0 (QM_ERR_INVALID otherwise); a_codes, b, c 16-byte and a_scales 2-byte
 * aligned.
 */
int qm_gemm_mxfp4_bf16_nn(const uint8_t* a_codes, const uint8_t* a_scales, const void* b, int64_t M, int64_t N, int64_t K,
                          float alpha, void* c, int c_dtype, void* stream);

/*
 * qm_gemm_mxfp4_tn for callers that cannot allocate (code under HIP graph capture, serving loops, harnesses that forbid
 * hipMalloc).  It has no counterpart in the reference.  Same arguments and the same results, bit for bit, as
 * qm_gemm_mxfp4_tn offered qm_gemm_workspace_bytes(M, N, K) bytes of workspace; the split-K partial sums live in a
 * device array built into the library (QM_GEMM_NOALLOC_SCRATCH_BYTES per GPU, held until the process ends) instead.
 * A shape whose partial sums need more is rejected with QM_ERR_INVALID.  Nothing in the array has to start at zero
 * (every partial sum that is read has been written by the same call), but every call on a GPU uses that GPU's one
 * array: calls that overlap on one GPU (two streams, two threads) race.  Allocates nothing, frees nothing --
 * with one proviso about the HIP runtime: the device address of the array is looked up on a device's first use, and
 * that lookup is when the runtime places this library's device image (the array included) in that GPU's memory.
 * qm_gemm_noalloc_prepare() performs the lookup for the current device and nothing else: call it once per device,
 * outside any stream capture, before the first call that must not allocate (a first qm_gemm_mxfp4_tn_noalloc call
 * without it does the lookup itself).  Every later call on that device touches no allocator of any kind.
 */
#define QM_GEMM_NOALLOC_SCRATCH_BYTES ((size_t)64 << 20)
size_t qm_gemm_noalloc_scratch_bytes(void);
int qm_gemm_noalloc_prepare(void);
int qm_gemm_mxfp4_tn_noalloc(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                             const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c,
                             int c_dtype, int a_layout, int b_layout, void* stream);

/*
 * Measurement aid, no counterpart in the reference: the block-scaled FP4 matrix instruction of the product above in a
 * loop without memory traffic, on operand bytes taken from `operands` (one workgroup of four waves per CU, each wave
 * 16 instructions of 32 x 32 x 64 per iteration).  The rate it reaches on the bytes of real operands is the ceiling
 * the chip's power limit leaves for qm_gemm_mxfp4_tn; bench.py reports both.  Returns the number of matrix
 * instructions issued (each 2 * 32 * 32 * 64 flop), or a negative value on rejected arguments / launch failure.
 *   operands: at least 32 KiB per CU, 16-byte aligned; sink: at least 1 KiB per CU (receives checksums).
 */
int64_t qm_diag_mfma_only(const uint8_t* operands, size_t operand_bytes, float* sink, size_t sink_bytes, int iters,
                          void* stream);
/*
 * Measurement aid, no counterpart in the reference: one launch of an instantiation of the product's persistent tile kernel
 * (bf16 output, arguments as qm_gemm_mxfp4_tn) that also records the shader clock, per workgroup, at its entry, at the
 * start of its tile loop, and after every tile's K loop and epilogue (up to 15 tiles): QM_DIAG_PHASE_STAMPS 64-bit values
 * per workgroup into `stamps` (DEVICE memory, stamps_bytes >= workgroups * QM_DIAG_PHASE_STAMPS * 8; one workgroup per
 * CU or per tile, whichever is fewer).  Where the time of a tile goes -- K steps against the epilogue, during which no
 * matrix instruction runs -- is read from the differences; bench.py --gemm-phases prints them.  c receives the product.
 * maskbits (optional, [M, N/8], 4-byte aligned): stamp the instantiation whose epilogue carries the masked inverse rotation
 * of qm_gemm_mxfp4_tn_rotated (no sign flips, bf16 scale); c then receives the rotated product.
 * Serves M, N multiples of 64 and >= 256, K % 512 == 0.  Returns the number of workgroups launched, or a negative
 * status.
 */
#define QM_DIAG_PHASE_STAMPS 32
int qm_diag_gemm_tile_phases(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                             int64_t M, int64_t N, int64_t K, float alpha, void* c, int a_layout, int b_layout,
                             const uint8_t* maskbits, uint64_t* stamps, size_t stamps_bytes, void* stream);

/*
 * c = masked inverse rotation of (alpha * A B^T): qm_gemm_mxfp4_tn with a bf16 result followed by qm_masked_hadamard_bwd
 * (Hadamard block 32 along N, bf16 in and out), the pair a gradient product and the forward quantizer's straight-through
 * backward form in the layer's backward pass (src/models/quantization/backward.py:62,71-83 feeding
 * quantizers/mxfp4.py:143-146), as ONE launch: the persistent product kernel rounds its tile to bf16, multiplies it by the
 * mask and rotates it on the matrix pipe before storing it, so the rotated-basis gradient never travels through memory.
 * Same values as the two calls except that a group's 32 terms are added in the matrix instruction's order (fp32 sums of
 * bf16 values: a few results in 10^4 differ in the last bf16 bit).
 *   maskbits     [M, N/8] clip-mask bits of the forward quantizer (bit n % 8 of byte n / 8), 4-byte aligned; sign_bits,
 *                scale_dtype as for qm_masked_hadamard_bwd with hadamard_dim 32
 *   Served shapes: those of the persistent kernel without a cut into K ranges -- qm_gemm_fuses_rotation() tells (M, N
 *   multiples of 64 and >= 256, K % 128 == 0 and > 768, scale arrays 16-byte aligned when K % 512 == 0, few enough output
 *   tiles that no workspace would be used); anything else returns QM_ERR_INVALID and the caller makes the two calls.
 */
int qm_gemm_fuses_rotation(const uint8_t* a_scales, const uint8_t* b_scales, int64_t M, int64_t N, int64_t K);
int qm_gemm_mxfp4_tn_rotated(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                             int64_t M, int64_t N, int64_t K, float alpha, void* c, int a_layout, int b_layout,
                             const uint8_t* maskbits, const uint32_t* sign_bits, int scale_dtype, void* stream);

/*
 * out = ((g * mask).view(-1, hd)) @ H^T: the straight-through backward of the forward quantizer,
 * QuestMXFP4QuantizerFn.backward (src/models/quantization/quantizers/mxfp4.py:143-146); with
 * maskbits == NULL it is AlbertTsengQuantizerFn.backward (mxfp4.py:31-34).
 *   scale_dtype  dtype whose rounding of hd^-1/2 the matrix H carries
 */
int qm_masked_hadamard_bwd(const void* g, int g_dtype, int64_t rows, int64_t cols,
                           int hadamard_dim, int scale_dtype, const uint32_t* sign_bits,
                           const uint8_t* maskbits, void* out, int out_dtype, void* stream);

/* out[r, c] = e2m1(code) * post * 2^(scale-127); the tensor the reference's pseudo-quantizer returns */
int qm_dequantize_mxfp4(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C,
                        float post, void* out, int out_dtype, void* stream);

/*
 * Whole-layer entry points: one call issues every launch of a Quartet linear's forward or backward pass (the
 * per-kernel entry points above, in order), so the host pays one foreign call instead of three / eight.
 *
 * A packed operand is one caller-owned, 256-byte aligned buffer of qm_packed_operand_bytes(rows, cols) bytes holding,
 * at the offsets qm_packed_operand_offsets reports, the codes [rows, cols/2], E8M0 scales [rows, cols/32] and
 * clip-mask bits [rows, cols/8] of a quantized [rows, cols] tensor -- the three tensors per operand that
 * notebooks/benchmark_mxfp4.ipynb's CudaGemm keeps for backward (ctx.save_for_backward in its forward).
 *
 * qm_linear_forward = QuestMXFP4QuantizerFn.forward on x and W (quantizers/mxfp4.py:129-140) followed by
 * QEQWtt_QEtQXttFn.forward (src/models/quantization/backward.py:59-62):
 *   x [T, I], w [O, I] -> y [T, O] = Q(x) Q(w)^T; packed_x ([T, I]) and packed_w ([O, I]) receive the packed
 *   operands the backward pass needs.  packed_flags & QM_W_IS_PACKED: packed_w already holds Q(w) from an earlier
 *   call with the same w, signs and layout, and w is not read (W changes only at the optimizer step,
 *   src/optim/base.py:188-207, so the micro-steps of a gradient accumulation quantize it once).
 *   packed_flags & QM_X_IS_PACKED: packed_x already holds Q(x), written by one of the fused producers below, and x is
 *   not read.
 * qm_linear_backward = QEQWtt_QEtQXttFn.backward (backward.py:64-85) with the straight-through backward of both
 * forward quantizers (mxfp4.py:143-146) applied: e [T, O] -> gx [T, I] of mid_dtype, gw [O, I] of gw_dtype.
 *   g_mode            QM_ABSMAX_SR or QM_ABSMAX_RTN (AlbertTsengQuantizer stochastic or not)
 *   seeds             HOST pointer to four seeds, for the quantizations of e, Q(w)^T, e^T, Q(x)^T in that order
 *   x_val_dtype, w_val_dtype   dtypes the reference would hold the de-quantized x and w in
 *   x_scale_dtype, w_scale_dtype  dtypes whose rounding of hd^-1/2 the forward quantizers' matrices carry in backward
 *   workspace         qm_linear_backward_workspace_bytes(T, I, O, mid_dtype) bytes of scratch, 256-byte aligned
 *   gw_dtype          dtype of gw: mid_dtype, or QM_F32 with a bf16 mid_dtype -- then gw holds the bf16-rounded values
 *                     widened to fp32, i.e. what autograd's cast of a bf16 gradient to an fp32 weight's dtype produces
 *   g_matrix          NULL, or a DEVICE pointer to the gradient quantizer's dense rotation ([32][32] fp32, as for
 *                     qm_quantize_mxfp4_dense; AlbertTsengQuantizer with rerotate="O32"): replaces hd_g / signs_g in the
 *                     four gradient quantizations; needs hd_g == 32 and T, I, O multiples of 128
 *   rotated_flags     QM_GX_ROTATED: gx receives the gradient w.r.t. the activation quantizer's rotated output (the first
 *                     product, B3) and its straight-through backward is left to the caller, who folds it into the
 *                     next kernel (maskbits argument of qm_rmsnorm_backward / qm_swiglu_backward) or, for a forward
 *                     quantizer that holds a dense rotation, applies mask and transposed matrix itself; needs hd_x == 32.
 *                     QM_GW_ROTATED: the same for gw and the weight quantizer (second product, B6; gw_dtype == mid_dtype)
 * codes_layout applies to every packed tensor inside; QM_LAYOUT_TILED needs T, I, O multiples of 128 and at
 * least 256, and all Hadamard blocks 32.  T, I, O must be multiples of 32 for the backward pass.
 * Where a gradient product runs as qm_gemm_fuses_rotation describes (bf16 mid_dtype, Hadamard block 32, for gw also
 * gw_dtype == mid_dtype), the forward quantizer's masked inverse rotation is applied in that product's epilogue
 * (qm_gemm_mxfp4_tn_rotated) and the product is not staged in the workspace.  Where a gradient product is cut into K
 * ranges (Hadamard block 32, any mid_dtype / gw_dtype), the rotation is applied by the ordered reduction of the ranges,
 * with the arithmetic and roundings of the separate launches.  Elsewhere it is a launch of its own.
 */
size_t qm_packed_operand_bytes(int64_t rows, int64_t cols);
/* offsets: HOST array of three (codes, scales, mask bits); returns 0, or QM_ERR_INVALID unless cols % 32 == 0 */
int qm_packed_operand_offsets(int64_t rows, int64_t cols, size_t* offsets);
size_t qm_linear_backward_workspace_bytes(int64_t T, int64_t I, int64_t O, int mid_dtype);
int qm_linear_forward(const void* x, int x_dtype, const void* w, int w_dtype, int64_t T, int64_t I, int64_t O,
                      int hd_x, const uint32_t* signs_x, int hd_w, const uint32_t* signs_w, void* packed_x,
                      size_t packed_x_bytes, void* packed_w, size_t packed_w_bytes, int packed_flags, void* y,
                      int y_dtype, int codes_layout, void* stream);
int qm_linear_backward(const void* e, int e_dtype, int64_t T, int64_t I, int64_t O, const void* packed_x,
                       const void* packed_w, int hd_x, const uint32_t* signs_x, int hd_w, const uint32_t* signs_w,
                       int hd_g, const uint32_t* signs_g, int g_mode, const uint64_t* seeds, int x_val_dtype,
                       int w_val_dtype, int mid_dtype, int x_scale_dtype, int w_scale_dtype, void* workspace,
                       size_t workspace_bytes, void* gx, void* gw, int gw_dtype, int codes_layout, int rotated_flags,
                       const float* g_matrix, void* stream);
/*
 * qm_linear_backward for callers that replay the step from a captured HIP graph.  It has no counterpart in the reference
 * (whose stochastic rounding draws a fresh host seed per call, mxfp4_triton.py:196-199, which a captured graph would
 * freeze).  seed_base: NULL (then exactly qm_linear_backward), or a DEVICE pointer, 8-byte aligned, to one 64-bit value
 * that the four gradient quantizations read when they run and add to their seed: a graph that also contains a kernel
 * incrementing that value draws fresh random streams on every replay.  With the value v the results equal those of
 * qm_linear_backward with seeds[i] + v.  Needs the layout the layer's production path uses (QM_LAYOUT_TILED, Hadamard
 * blocks 32, T, I, O multiples of 128, g_matrix == NULL); the sign words stay host values.
 */
int qm_linear_backward_seeded(const void* e, int e_dtype, int64_t T, int64_t I, int64_t O, const void* packed_x,
                              const void* packed_w, int hd_x, const uint32_t* signs_x, int hd_w, const uint32_t* signs_w,
                              int hd_g, const uint32_t* signs_g, int g_mode, const uint64_t* seeds, int x_val_dtype,
                              int w_val_dtype, int mid_dtype, int x_scale_dtype, int w_scale_dtype, void* workspace,
                              size_t workspace_bytes, void* gx, void* gw, int gw_dtype, int codes_layout, int rotated_flags,
                              const float* g_matrix, const uint64_t* seed_base, void* stream);

/*
 * Producers fused into the activation quantizer.  The tensor the model would hand to a quantized linear is computed
 * group by group inside the quantizer kernel and never written; the result is a packed operand buffer (layout as
 * above) that qm_linear_forward consumes with QM_X_IS_PACKED and qm_linear_backward reads as packed_x.  Hadamard block
 * 32, QM_QUEST_RTN with clip mask (QuestMXFP4QuantizerFn.forward, quantizers/mxfp4.py:129-140).
 *
 * qm_rmsnorm_quantize_mxfp4: RMSNorm.forward (src/models/llama.py:64-75) in front of c_attn / w12 (llama.py:170-171):
 *   Q((x.float() * rsqrt(mean(x^2, -1) + eps)).type_as(x) * gain), x [rows, cols], gain fp32 [cols]; the product with
 *   the fp32 gain is fp32, so the quantizer runs as on an fp32 tensor.  factor [rows] fp32 receives
 *   rsqrt(mean(x^2) + eps) for the backward pass.  add (optional; x fp32, add of add_dtype): the block's residual sum in
 *   front of the norm (x + attn(...), x + mlp(...), llama.py:170-171) is formed here: the norm's input is x + add, which
 *   is also written to x_sum [rows, cols] fp32 for the rest of the model.
 * qm_swiglu_quantize_mxfp4: the SwiGLU product in front of the MLP's c_proj (llama.py:113-114):
 *   Q(silu(up) * gate) with h12 [rows, 2 hidden] = (up, gate) the fused w12 output; a bf16 h12 rounds silu and the
 *   product to bf16 as torch's bf16 ops do, and the quantizer runs as on a tensor of h12's dtype.
 * qm_rmsnorm_backward: autograd of the RMSNorm line above: gy [rows, cols] (gradient w.r.t. the normalised, scaled
 *   tensor) -> dx [rows, cols] of x's dtype and dgain fp32 [cols] (summed over rows in a fixed order).  cols <= 8192.
 *   workspace: qm_rmsnorm_backward_workspace_bytes(rows, cols) bytes, 16-byte aligned.  skip (optional, [rows, cols] of
 *   x's dtype): the gradient that reaches x past the norm (x + f(norm(x)), llama.py:170-171); dx = skip + the norm's
 *   gradient, the sum autograd would form in a pass of its own.  dx_bf16 (optional): dx rounded to bf16 as well, the
 *   gradient of a bf16 `add` of qm_rmsnorm_quantize_mxfp4.
 * qm_swiglu_backward: autograd of silu(up) * gate: g [rows, hidden] -> d_h12 [rows, 2 hidden] of h12's dtype.
 *   Both backward kernels take the gradient either as it is (maskbits == NULL) or still in the rotated basis of the
 *   layer's activation quantizer (qm_linear_backward with QM_GX_ROTATED): then maskbits [rows, cols/8] (the mask region of
 *   the layer's packed_x; 4-byte aligned for qm_rmsnorm_backward), sign_bits and scale_dtype describe that quantizer, and the masked inverse rotation of
 *   qm_masked_hadamard_bwd (same operations, same bits, rounded to the gradient's dtype) is applied on the fly.
 * codes_layout QM_LAYOUT_TILED needs rows % 16 == 0 and cols (hidden) % 128 == 0; cols (hidden) % 32 == 0 always.
 */
int qm_rmsnorm_quantize_mxfp4(const void* x, int x_dtype, const void* add, int add_dtype, void* x_sum,
                              const float* gain, float eps, int64_t rows, int64_t cols, const uint32_t* sign_bits,
                              void* packed, size_t packed_bytes, float* factor, int codes_layout, void* stream);
int qm_swiglu_quantize_mxfp4(const void* h12, int dtype, int64_t rows, int64_t hidden, const uint32_t* sign_bits,
                             void* packed, size_t packed_bytes, int codes_layout, void* stream);
size_t qm_rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols);
int qm_rmsnorm_backward(const void* gy, int gy_dtype, const void* x, int x_dtype, const float* gain,
                        const float* factor, int64_t rows, int64_t cols, const uint8_t* maskbits,
                        const uint32_t* sign_bits, int scale_dtype, const void* skip, void* dx, void* dx_bf16,
                        float* dgain, void* workspace, size_t workspace_bytes, void* stream);
int qm_swiglu_backward(const void* g, int g_dtype, const void* h12, int dtype, int64_t rows, int64_t hidden,
                       const uint8_t* maskbits, const uint32_t* sign_bits, int scale_dtype, void* d_h12,
                       void* stream);

/*
 * Rotary position embedding around the attention that sits between two quantized linears (apply_rotary_emb,
 * src/models/llama.py:43-61, called at llama.py:141-143 on the split of c_attn's output).
 * qm_rope_split_qkv: qkv [rows, 3 n_embd] = (q, k, v) -> q, k, v [rows, n_embd] of out_dtype; in every head of q and k
 *   the pairs (2i, 2i+1) are rotated by the angle of table[r % seq_len, i] = (cos, sin), in fp32 with every product and
 *   sum rounded (the reference's op-by-op arithmetic); v is copied (converted).  table: fp32 [seq_len, head_dim/2, 2].
 * qm_rope_merge_qkv_grad: the backward pass: gradients dq, dk, dv [rows, n_embd] of grad_dtype -> d_qkv [rows, 3 n_embd]
 *   of out_dtype, dq and dk rotated by the negative angle.
 * head_dim % 8 == 0, n_embd % head_dim == 0.
 */
int qm_rope_split_qkv(const void* qkv, int qkv_dtype, int64_t rows, int64_t seq_len, int64_t n_embd, int head_dim,
                      const float* table, void* q, void* k, void* v, int out_dtype, void* stream);
int qm_rope_merge_qkv_grad(const void* dq, const void* dk, const void* dv, int grad_dtype, int64_t rows, int64_t seq_len,
                           int64_t n_embd, int head_dim, const float* table, void* d_qkv, int out_dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* QUARTET_HIP_H */
