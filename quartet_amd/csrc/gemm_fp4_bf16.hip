// MXFP4 x bf16 "NN" GEMM: the two gradient products of the scheme that quantizes only the error signal.
//
//   C[m, n] = alpha * sum_k A[m, k] * B[k, n]
//
// A: packed E2M1 codes [M, K/2] (element 2i in the low nibble of byte i) + E8M0 scales [M, K/32], row-major;
// B: bf16 [K, N] row-major (n contiguous) -- the layer's saved, unquantized operand exactly as it lies in memory.
// Replaces, in QEW_QEtXFn.backward (src/models/quantization/backward.py:31-43 of the reference),
//   grad_x = F.linear(Q(e), w.T)                      A = Q(e)   [T, O], B = w [O, I]
//   grad_w = einsum("ib,bj->ij", Q(e^T), x)           A = Q(e^T) [O, T], B = x [T, I]
// which the reference runs as library bf16 GEMMs on a de-quantized copy of Q(e) (and, for the second, after an explicit
// transposed copy of e).  Here Q(e) stays packed: 0.53 B/elt instead of 2, no de-quantized tensor in HBM.
//
// There is no matrix instruction that takes FP4 on one side and bf16 on the other, so the codes are decoded to bf16 in
// registers (v_cvt_scalef32_pk_bf16_fp4: one byte -> two bf16, times the group's power-of-two scale, exact) and the
// product runs on v_mfma_f32_32x32x16_bf16 with fp32 accumulation.
//
// Operand fetch.  The instruction wants, from both operands, eight consecutive-k values per lane.
//   A is packed along k: lane (row l%32, half h = l/32) reads the 16 code bytes of MX group h of the K step (64 values per
//   step) and its scale byte; dword s of those bytes decodes to the lane's share of matrix instruction s = 0..3.  The
//   contraction index is therefore consumed in the order k = 32 h + 8 s + t (h: lane half, t: slot within the lane).
//   B has k as its *strided* index.  Its tile goes to LDS as it is ([k][n], n contiguous) and ds_read_b64_tr_b16 transposes
//   on the way out: a group of 16 lanes pointing at a 4 (k) x 16 (n) block receives, lane = n, the four k values of its
//   column.  Two such reads give a lane the eight k of one instruction, in the same k order as A.
//   LDS rows of B are 256 bytes = all 64 banks; the 16-byte piece p of row k is stored at p ^ (4 (k & 3)), so that the four
//   rows one lane group reads fall on different banks (applied when the tile is written).
//
// Tile: 128 x 128 per workgroup, four waves of 64 x 64 (2 x 2 blocks of 32 x 32, 64 accumulator registers), K step 64,
// operands staged global -> registers -> LDS, double buffered, one barrier per step; two or three workgroups share a CU.
// B is fed as the instruction's first operand, so a lane's accumulator quads run along n and leave as 8-byte (bf16) or
// 16-byte (fp32) pieces of a row.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qm_kernels.h"
#include "qm_math.h"

namespace qm {

namespace {

typedef short v4s __attribute__((ext_vector_type(4)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));

constexpr int kTM = 128, kTN = 128, kTK = 64;
constexpr int kACodeBytes = kTM * (kTK / 2);   // 4 KiB: [128 rows][32 bytes]
constexpr int kAScaleBytes = kTM * 2;           // [128 rows][2 groups]
constexpr int kBBytes = kTK * kTN * 2;          // 16 KiB: [64 k][256 bytes]
constexpr int kStage = kACodeBytes + kAScaleBytes + kBBytes;
constexpr int kSmem = 2 * kStage;

// same tile walk as the FP4 x FP4 kernels: workgroup ids are dealt round-robin to the 8 XCDs; each XCD gets a contiguous
// run of tiles that walks 4-row groups column by column, so the tiles sharing an L2 share A and B panels
__device__ __forceinline__ void tile_of_block_nn(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
    const int total = tiles_m * tiles_n;
    int t = bid;
    if ((total & 7) == 0) t = (bid & 7) * (total >> 3) + (bid >> 3);
    constexpr int GM = 4;
    const int per_group = GM * tiles_n;
    const int group = t / per_group;
    const int first_m = group * GM;
    const int gm = (tiles_m - first_m) < GM ? (tiles_m - first_m) : GM;
    const int r = t - group * per_group;
    tm = first_m + r % gm;
    tn = r / gm;
}

template <typename OutT>
__global__ __launch_bounds__(256, 2) void gemm_fp4_bf16_nn_kernel(const uint8_t* __restrict__ a_codes,
                                                                  const uint8_t* __restrict__ a_scales,
                                                                  const uint16_t* __restrict__ b, int M, int N, int K,
                                                                  float alpha, OutT* __restrict__ c) {
    extern __shared__ uint8_t smem_nn[];
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, half = lane >> 5;
    int tm, tn;
    tile_of_block_nn((int)blockIdx.x, (M + kTM - 1) / kTM, (N + kTN - 1) / kTN, tm, tn);
    const int64_t m0 = (int64_t)tm * kTM, n0 = (int64_t)tn * kTN;
    const int64_t code_pitch = K / 2, groups = K / 32;
    const int nk = K / kTK;

    // ---- global -> registers: what this thread fetches per K step --------------------------------------------------
    // A codes: row tid/2, 16-byte half tid%2 (rows beyond M read the last row; their results are dropped)
    const int a_row = tid >> 1, a_half = tid & 1;
    const int64_t a_grow = m0 + a_row < M ? m0 + a_row : (int64_t)M - 1;
    const uint8_t* a_src = a_codes + a_grow * code_pitch + a_half * 16;
    // A scales: threads 0..127, the row's two bytes of the step
    const int64_t s_grow = m0 + (tid & 127) < M ? m0 + (tid & 127) : (int64_t)M - 1;
    const uint8_t* s_src = a_scales + s_grow * groups;
    // B: four 16-byte pieces; piece id p = tid + 256 c: row p / 16, piece p % 16 (columns beyond N read as zero)
    const int b_piece = tid & 15, b_row0 = tid >> 4;  // rows b_row0 + 16 c
    const bool b_in = n0 + b_piece * 8 < N;           // N % 8 == 0: a piece is inside or outside as a whole
    const uint16_t* b_src = b + (int64_t)b_row0 * N + n0 + b_piece * 8;

    uint4 ra, rb[4];
    uint32_t rs = 0u;
    auto load_global = [&](int ks) {
        ra = *reinterpret_cast<const uint4*>(a_src + (int64_t)ks * (kTK / 2));
        if (tid < kTM) rs = *reinterpret_cast<const uint16_t*>(s_src + (int64_t)ks * 2);
#pragma unroll
        for (int cidx = 0; cidx < 4; ++cidx) {
            rb[cidx] = make_uint4(0, 0, 0, 0);
            if (b_in) rb[cidx] = *reinterpret_cast<const uint4*>(b_src + ((int64_t)ks * kTK + 16 * cidx) * N);
        }
    };
    auto store_lds = [&](int buf) {
        uint8_t* st = smem_nn + buf * kStage;
        *reinterpret_cast<uint4*>(st + a_row * 32 + a_half * 16) = ra;
        if (tid < kTM) *reinterpret_cast<uint16_t*>(st + kACodeBytes + tid * 2) = (uint16_t)rs;
        uint8_t* sb = st + kACodeBytes + kAScaleBytes;
#pragma unroll
        for (int cidx = 0; cidx < 4; ++cidx) {
            const int row = b_row0 + 16 * cidx;
            *reinterpret_cast<uint4*>(sb + row * 256 + ((b_piece ^ (4 * (row & 3))) * 16)) = rb[cidx];
        }
    };

    // ---- LDS -> registers: per-lane offsets ------------------------------------------------------------------------
    // A: row wm*64 + i*32 + lrow, MX group `half` of the step
    const int a_off = (wm * 64 + lrow) * 32 + half * 16;
    const int as_off = kACodeBytes + (wm * 64 + lrow) * 2 + half;
    // B transposing read: lane group g = lane/16 covers n-half g&1 of a 32-column block for lane half g>>1 (= `half`);
    // within the group lane r points at row (r / 4) of the four and at the 8-byte chunk r % 4 of the group's 32 bytes
    const int r16 = lane & 15, nh = (lane >> 4) & 1;
    const int b_krow = 32 * half + (r16 >> 2);                     // + 8 s + 4 rd
    const int b_byte = (wn * 64 + 16 * nh + 4 * (r16 & 3)) * 2;    // + 64 j : byte offset of the chunk within its row
    // the swizzle depends on (row & 3) = (r16 >> 2) & 3 only: 8 s + 4 rd + 32 half leave it unchanged
    const int b_swz = 4 * ((r16 >> 2) & 3);
    int b_off[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int byte = b_byte + 64 * j;
        b_off[j] = kACodeBytes + kAScaleBytes + b_krow * 256 + (((byte >> 4) ^ b_swz) << 4) + (byte & 15);
    }

    v16f acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    load_global(0);
    store_lds(0);
    __syncthreads();

    for (int ks = 0; ks < nk; ++ks) {
        const int buf = ks & 1;
        if (ks + 1 < nk) load_global(ks + 1);
        const uint8_t* st = smem_nn + buf * kStage;
        // A fragments: decode the lane's 32 codes of each row block; instruction s takes dword s
        v8bf af[2][4];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const uint4 q = *reinterpret_cast<const uint4*>(st + a_off + i * 32 * 32);
            const uint32_t sc = *(st + as_off + i * 32 * 2);
            const float scale = u2f(sc << 23);   // E8M0 -> 2^(sc - 127); byte 0 reads as 0 instead of 2^-127
            const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[s], scale, 0);
                const v2bf p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[s], scale, 1);
                const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[s], scale, 2);
                const v2bf p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[s], scale, 3);
                af[i][s] = v8bf{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
            }
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            v8bf bf[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                typedef v4s __attribute__((address_space(3))) * lds_v4s;
                const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(st + b_off[j] + (8 * s) * 256));
                const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(st + b_off[j] + (8 * s + 4) * 256));
                typedef short v8s __attribute__((ext_vector_type(8)));
                bf[j] = __builtin_bit_cast(v8bf, v8s{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[j], af[i][s], acc[i][j], 0, 0, 0);
        }
        if (ks + 1 < nk) store_lds(buf ^ 1);
        __syncthreads();
    }

    // epilogue: element e of block (i, j) is n = 8 (e/4) + 4 half + e%4 of the block, row m = lrow
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int64_t row = m0 + wm * 64 + i * 32 + lrow;
        if (row >= M) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int64_t col = n0 + wn * 64 + j * 32 + 8 * qd + 4 * half;
                if (col >= N) continue;   // N % 4 == 0: the quad is inside or outside as a whole
                const float v0 = acc[i][j][4 * qd] * alpha, v1 = acc[i][j][4 * qd + 1] * alpha;
                const float v2 = acc[i][j][4 * qd + 2] * alpha, v3 = acc[i][j][4 * qd + 3] * alpha;
                if constexpr (sizeof(OutT) == 2) {
                    const v2bf p0 = __builtin_convertvector(v2f{v0, v1}, v2bf);
                    const v2bf p1 = __builtin_convertvector(v2f{v2, v3}, v2bf);
                    *reinterpret_cast<uint2*>(c + row * N + col) =
                        make_uint2(__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1));
                } else {
                    *reinterpret_cast<float4*>(c + row * N + col) = make_float4(v0, v1, v2, v3);
                }
            }
    }
}

}  // namespace

bool gemm_fp4_bf16_nn_supported(int64_t M, int64_t N, int64_t K) {
    return M > 0 && N > 0 && K > 0 && K % kTK == 0 && N % 8 == 0 && M < (1 << 30) && N < (1 << 30) && K < (1 << 30) &&
           ((M + kTM - 1) / kTM) * ((N + kTN - 1) / kTN) < (int64_t)1 << 31;
}

hipError_t gemm_fp4_bf16_nn(const uint8_t* a_codes, const uint8_t* a_scales, const void* b, int64_t M, int64_t N, int64_t K,
                            float alpha, void* c, int c_dtype, hipStream_t stream) {
    if (M == 0 || N == 0) return hipSuccess;
    if (!gemm_fp4_bf16_nn_supported(M, N, K)) return hipErrorInvalidValue;
    dim3 grid((unsigned)(((M + kTM - 1) / kTM) * ((N + kTN - 1) / kTN))), block(256);
    if (c_dtype == BF16)
        gemm_fp4_bf16_nn_kernel<uint16_t><<<grid, block, kSmem, stream>>>(a_codes, a_scales, static_cast<const uint16_t*>(b), (int)M,
                                                                          (int)N, (int)K, alpha, static_cast<uint16_t*>(c));
    else
        gemm_fp4_bf16_nn_kernel<float><<<grid, block, kSmem, stream>>>(a_codes, a_scales, static_cast<const uint16_t*>(b), (int)M, (int)N,
                                                                       (int)K, alpha, static_cast<float*>(c));
    return hipGetLastError();
}

}  // namespace qm
