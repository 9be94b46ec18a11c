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

#include <atomic>
#include <type_traits>

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


// ---- large-tile variant: 256 x 256 per workgroup, one wave per SIMD owning 128 x 128 ---------------------------------
// For products with at least one full tile in each direction.  Four waves x (4 x 4 blocks of 32 x 32) = 256 accumulator
// registers; per K step of 64 a wave issues 64 matrix instructions against 4 code reads, 32 transposing reads and 64
// decode instructions, so LDS and the vector ALU stay well below the matrix pipe's time.  Operands go global -> LDS
// directly (global_load_lds_dwordx4) into a ring of three stages, requested two K steps ahead; the B swizzle is applied
// on the global-address side of those loads.  Scale bytes go global -> registers directly (one 16-bit load per row block
// and step: a lane keeps the two E8M0 bytes of its row's step and picks its half's).  One barrier per K step.
constexpr int kBM = 256, kBN = 256;
constexpr int kBigA = kBM * (kTK / 2);       // 8 KiB of codes per stage: [256 rows][32 bytes]
constexpr int kBigB = kTK * kBN * 2;         // 32 KiB: [64 k][512 bytes]
constexpr int kBigStage = kBigA + kBigB;
constexpr int kBigStages = 3;
constexpr int kBigSmem = kBigStages * kBigStage;   // 120 KiB
constexpr int kBigLoads = 14;                // VMEM instructions per wave per K step: 2 (A) + 8 (B) + 4 (scales)

// global -> LDS without passing through registers; issued from assembly so that the compiler's wait-count insertion
// does not treat every later LDS read as depending on it (the kernel waits explicitly for the stage it is about to read).
// LDS destination = lds_base (wave-uniform, through M0) + lane * 16.
__device__ __forceinline__ void dma_b128(const uint8_t* base, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(lds_base) : "memory");
}
__device__ __forceinline__ void dma_b128_v(const uint8_t* gsrc, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(gsrc), "s"(lds_base) : "memory");
}
__device__ __forceinline__ uint32_t load_u16_async(const uint8_t* base, uint32_t lane_off) {
    uint32_t v;
    asm volatile("global_load_ushort %0, %1, %2" : "=v"(v) : "v"(lane_off), "s"(base) : "memory");
    return v;
}
constexpr int vmcnt_only(int n) { return 0x0f70 | (n & 0xf) | ((n >> 4) << 14); }

template <typename OutT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_fp4_bf16_nn_big_kernel(
    const uint8_t* __restrict__ a_codes, const uint8_t* __restrict__ a_scales, const uint16_t* __restrict__ b, int M, int N, int K,
    float alpha, OutT* __restrict__ c) {
    extern __shared__ uint8_t smem_nn[];
    const uint32_t smem_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem_nn;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, half = lane >> 5;
    int tm, tn;
    tile_of_block_nn((int)blockIdx.x, (M + kBM - 1) / kBM, (N + kBN - 1) / kBN, tm, tn);
    const int64_t m0 = (int64_t)tm * kBM, n0 = (int64_t)tn * kBN;
    const int64_t code_pitch = K / 2, groups = K / 32;
    const int nk = K / kTK;

    // ---- what this wave requests per K step ---------------------------------------------------------------------------
    // A codes: two wave-loads of 32 rows x 32 bytes (rows wave*64 + 32 v + lane/2, 16-byte half lane%2); rows beyond M
    // read the last row, their results are dropped
    const uint8_t* a_src[2];
#pragma unroll
    for (int v = 0; v < 2; ++v) {
        int64_t row = m0 + wave * 64 + 32 * v + (lane >> 1);
        row = row < M ? row : (int64_t)M - 1;
        a_src[v] = a_codes + row * code_pitch + (lane & 1) * 16;
    }
    // B: eight wave-loads of 2 rows x 512 bytes (rows wave*16 + 2 u + lane/32).  LDS slot lane%32 of a row holds the
    // logical 16-byte piece (lane%32) ^ 4 (row & 3); row & 3 = 2 (u & 1) + lane/32.  Pieces beyond N read the row's last
    // piece instead (their columns are dropped).
    const int last_piece = (int)((N - n0 + 7) / 8) - 1;   // N % 8 == 0
    uint32_t b_lane[2];
#pragma unroll
    for (int par = 0; par < 2; ++par) {
        int piece = (lane & 31) ^ (4 * (2 * par + (lane >> 5)));
        piece = piece < last_piece ? piece : last_piece;
        b_lane[par] = (uint32_t)((lane >> 5) * N * 2 + piece * 16);
    }
    const uint8_t* b_base = reinterpret_cast<const uint8_t*>(b + (int64_t)(wave * 16) * N + n0);   // + (ks * 64 + 2 u) rows
    const int64_t b_row_bytes = (int64_t)N * 2;
    // scales: per row block i the two bytes of row wm*128 + i*32 + lrow at step ks
    uint32_t s_lane[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        int64_t row = m0 + wm * 128 + i * 32 + lrow;
        row = row < M ? row : (int64_t)M - 1;
        s_lane[i] = (uint32_t)(row * groups);
    }
    const uint32_t lds_a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_base + wave * 2048));
    const uint32_t lds_b = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_base + kBigA + wave * 8192));

    uint32_t sc[kBigStages][4] = {};
    auto issue = [&](int ks, int stage, uint32_t (&scs)[4]) {
        const int kk = ks < nk ? ks : nk - 1;   // past the end: a harmless repeat of the last step into a free stage
        const uint32_t sa = lds_a + stage * kBigStage, sb = lds_b + stage * kBigStage;
        dma_b128_v(a_src[0] + (int64_t)kk * 32, sa);
        dma_b128_v(a_src[1] + (int64_t)kk * 32, sa + 1024);
        const uint8_t* bs = b_base + (int64_t)kk * kTK * b_row_bytes;
#pragma unroll
        for (int u = 0; u < 8; ++u) dma_b128(bs + (int64_t)(2 * u) * b_row_bytes, b_lane[u & 1], sb + u * 1024);
        const uint8_t* ss = a_scales + (int64_t)kk * 2;
#pragma unroll
        for (int i = 0; i < 4; ++i) scs[i] = load_u16_async(ss, s_lane[i]);
    };

    // ---- LDS -> registers: per-lane offsets ---------------------------------------------------------------------------
    const int a_off = (wm * 128 + lrow) * 32 + half * 16;                 // + i * 1024
    const int r16 = lane & 15, nh = (lane >> 4) & 1;
    const int b_krow = 32 * half + (r16 >> 2);                            // + 8 s + 4 rd
    const int b_swz = 4 * ((r16 >> 2) & 3);
    int b_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int byte = (wn * 128 + j * 32 + 16 * nh + 4 * (r16 & 3)) * 2;
        b_off[j] = kBigA + b_krow * 512 + (((byte >> 4) ^ b_swz) << 4) + (byte & 15);
    }

    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

    auto compute = [&](int stage, uint32_t (&scs)[4]) {
        const uint8_t* st = smem_nn + stage * kBigStage;
        uint4 codes[4];
        float scale[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            codes[i] = *reinterpret_cast<const uint4*>(st + a_off + i * 1024);
            scale[i] = u2f(__builtin_amdgcn_ubfe(scs[i], (uint32_t)(8 * half), 8u) << 23);   // E8M0 -> 2^(byte - 127); byte 0 reads as 0
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            v8bf bf[4], af[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                typedef v4s __attribute__((address_space(3))) * lds_v4s;
                typedef short v8s __attribute__((ext_vector_type(8)));
                const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(st + b_off[j] + (8 * s) * 512));
                const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(st + b_off[j] + (8 * s + 4) * 512));
                bf[j] = __builtin_bit_cast(v8bf, v8s{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]});
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t w = s == 0 ? codes[i].x : (s == 1 ? codes[i].y : (s == 2 ? codes[i].z : codes[i].w));
                const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale[i], 0);
                const v2bf p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale[i], 1);
                const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale[i], 2);
                const v2bf p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale[i], 3);
                af[i] = v8bf{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
    };

    // One K step: wait for this wave's share of the stage (WAIT = how many younger loads may still be in flight: the 14
    // of the step after it), barrier (every wave's share has landed, and every wave has finished reading the stage about
    // to be refilled), request step ks + 2 into the stage freed by step ks - 1, then compute.
    // The scale loads write their registers when they land, not when they issue: a register whose value the compiler
    // considers dead would be handed to something else and then overwritten by the late load.  So the steps after the
    // main loop request nothing, and the final wait names every scale register.
    auto step = [&](int ks, auto stage_c, auto issue_c, auto wait_c) {
        constexpr int S = decltype(stage_c)::value;
        constexpr int WAIT = decltype(wait_c)::value;
        asm volatile("s_waitcnt vmcnt(%4)" : "+v"(sc[S][0]), "+v"(sc[S][1]), "+v"(sc[S][2]), "+v"(sc[S][3]) : "n"(WAIT) : "memory");
        __syncthreads();
        if constexpr (decltype(issue_c)::value) issue(ks + 2, (S + 2) % kBigStages, sc[(S + 2) % kBigStages]);
        compute(S, sc[S]);
    };
    using std::integral_constant;
    issue(0, 0, sc[0]);
    issue(1, 1, sc[1]);
    int ks = 0;
    for (; ks + 3 <= nk; ks += 3) {
        step(ks, integral_constant<int, 0>{}, std::true_type{}, integral_constant<int, kBigLoads>{});
        step(ks + 1, integral_constant<int, 1>{}, std::true_type{}, integral_constant<int, kBigLoads>{});
        step(ks + 2, integral_constant<int, 2>{}, std::true_type{}, integral_constant<int, kBigLoads>{});
    }
    // two sets of loads are in flight here (steps ks and ks + 1, real or repeats)
    if (ks < nk) step(ks, integral_constant<int, 0>{}, std::false_type{}, integral_constant<int, kBigLoads>{});
    if (ks + 1 < nk) step(ks + 1, integral_constant<int, 1>{}, std::false_type{}, integral_constant<int, 0>{});
    // direct-to-LDS loads must not outlive the workgroup's LDS allocation, nor scale loads their registers
    asm volatile("s_waitcnt vmcnt(0)"
                 : "+v"(sc[0][0]), "+v"(sc[0][1]), "+v"(sc[0][2]), "+v"(sc[0][3]), "+v"(sc[1][0]), "+v"(sc[1][1]), "+v"(sc[1][2]),
                   "+v"(sc[1][3]), "+v"(sc[2][0]), "+v"(sc[2][1]), "+v"(sc[2][2]), "+v"(sc[2][3])
                 :
                 : "memory");

    // epilogue: element e of block (i, j) is n = 8 (e/4) + 4 half + e%4 of the block, row m = lrow
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int64_t row = m0 + wm * 128 + i * 32 + lrow;
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int qd = 0; qd < 4; ++qd) {
                const int64_t col = n0 + wn * 128 + j * 32 + 8 * qd + 4 * half;
                if (row >= M || col >= N) continue;   // N % 4 == 0: the quad is inside or outside as a whole
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
    if (M >= kBM && N >= kBN) {
        // at least one full 256 x 256 tile in each direction: the large-tile kernel
        dim3 grid((unsigned)(((M + kBM - 1) / kBM) * ((N + kBN - 1) / kBN))), block(256);
        static std::atomic<bool> allowed16[64], allowed32[64];
        int dev = 0;
        hipError_t e = hipGetDevice(&dev);
        if (e != hipSuccess) return e;
        auto allow = [&](auto kern, std::atomic<bool>(&done)[64]) -> hipError_t {
            if (dev >= 0 && dev < 64 && done[dev].load(std::memory_order_acquire)) return hipSuccess;
            hipError_t r = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kBigSmem);
            if (r == hipSuccess && dev >= 0 && dev < 64) done[dev].store(true, std::memory_order_release);
            return r;
        };
        if (c_dtype == BF16) {
            auto kern = gemm_fp4_bf16_nn_big_kernel<uint16_t>;
            if ((e = allow(kern, allowed16)) != hipSuccess) return e;
            kern<<<grid, block, kBigSmem, stream>>>(a_codes, a_scales, static_cast<const uint16_t*>(b), (int)M, (int)N, (int)K, alpha,
                                                    static_cast<uint16_t*>(c));
        } else {
            auto kern = gemm_fp4_bf16_nn_big_kernel<float>;
            if ((e = allow(kern, allowed32)) != hipSuccess) return e;
            kern<<<grid, block, kBigSmem, stream>>>(a_codes, a_scales, static_cast<const uint16_t*>(b), (int)M, (int)N, (int)K, alpha,
                                                    static_cast<float*>(c));
        }
        return hipGetLastError();
    }
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
