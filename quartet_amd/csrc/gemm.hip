// MXFP4 x MXFP4 "TN" GEMM on gfx950's block-scaled FP4 MFMA.
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
// Three kernels, picked by shape in gemm_mxfp4_tn() at the end of the file:
//   gemm_mxfp4_tn_big4_kernel  M, N multiples of 64 and >= 256, K > 768 and K % 512 == 0, or another multiple of 128 whose
//                              last block of four K steps repeats (muted) at most a third as many steps as K has.
//                              Persistent, 256x256 macro tile, 4 waves x 128x128, operands global -> LDS directly into a
//                              4-stage ring, scales in blocks of four K steps, row-major or tiled code bytes, optional split-K.
//   gemm_mxfp4_tn_duo_kernel   same M, N, K % 128 == 0 and K <= 768, or K % 128 == 64 (row-major operands, any K >= 192):
//                              256x128 tiles, two workgroups per CU hiding each other's tile boundaries, scales per K step.
//   gemm_mxfp4_tn_kernel       any M, N and K % 32 == 0: 128x128 macro tile, 4 waves x 64x64, operands staged
//                              global -> registers -> LDS (rows padded from 64 to 80 bytes so the 16-byte fragment
//                              reads of 16 consecutive rows hit 64 distinct banks), double buffered.
// All keep fp32 accumulators in registers, use one barrier per K step and apply alpha in the epilogue.
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>
#include <utility>

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


// ---- large-tile kernel: 256 x 256 macro tile, one wave per SIMD owning 128 x 128 -----------------
// Requires M % 256 == 0, N % 256 == 0, K % 128 == 0.
//
// Per K step of 128 a wave issues 32 MFMAs (2 sub-steps x 4 x 4 tiles) against 16 fragment reads of
// 16 bytes.  Operands go global -> LDS directly (global_load_lds_dwordx4: each wave instruction drops
// 64 x 16 B contiguously into LDS, no staging registers, no ds_write), into a ring of four stages, so
// a tile is requested three K steps before it is consumed.  LDS rows are 64 bytes; the 16-byte column
// of (row, c) is stored at c ^ ((row >> 2) & 3), applied on the global-address side of the load and on
// the fragment read, which keeps the 16-byte fragment reads of 32 consecutive rows off each other's banks.
typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

// acc element e of a 32x32 tile is row 8*(e/4) + 4*half + e%4, column lane%32: per store instruction the
// two half-waves each write one 64-byte (bf16) row segment.  (Making a lane's 4 values contiguous along n by
// swapping the MFMA operand roles was measured slower: 64 scattered 8-byte pieces per instruction.)
// One accumulator register into a vector register, in program order: left to itself the compiler copies ten blocks of
// sixteen ahead of the first pass, and the 160 registers that takes push values the K loop needs out to scratch memory,
// whose reloads then wait for every operand load in flight (loads return in order).
__device__ __forceinline__ float acc_read(float a) {
    float v;
    asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(a));
    return v;
}
// The hazard recogniser does not look inside assembly statements: a matrix instruction's result may be read by a vector
// instruction only a number of wait states after it issued (19 for the sixteen-pass forms).  Every epilogue that reads
// accumulators through acc_read() starts with this, whatever the scheduler has put between the last product and it.
__device__ __forceinline__ void acc_settle() { asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory"); }
template <typename OutT, bool IN_ORDER = false>
__device__ __forceinline__ void store_tile(const v16f& t, float alpha, OutT* __restrict__ c, int64_t row0, int64_t col,
                                           int64_t N, int half) {
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
        const int64_t r = row0 + 8 * (e / 4) + 4 * half + (e & 3);
        const float v0 = (IN_ORDER ? acc_read(t[e]) : t[e]) * alpha, v1 = (IN_ORDER ? acc_read(t[e + 1]) : t[e + 1]) * alpha;
        if constexpr (sizeof(OutT) == 2) {
            // v_cvt_pk_bf16_f32: round-to-nearest-even, two values per instruction
            const v2bf p = __builtin_convertvector(v2f{v0, v1}, v2bf);
            const uint32_t bits = __builtin_bit_cast(uint32_t, p);
            c[r * N + col] = (uint16_t)(bits & 0xffffu);
            c[(r + 1) * N + col] = (uint16_t)(bits >> 16);
        } else {
            c[r * N + col] = v0;
            c[(r + 1) * N + col] = v1;
        }
    }
}

constexpr int kBigM = 256, kBigN = 256;
constexpr int kStages = 4;
constexpr int kBOff = kBigM * kRowBytes;

// Tile order: workgroup ids are dealt round-robin to the 8 XCDs by the hardware; give each XCD a
// contiguous run of tiles in an order that walks 4-row groups column by column, so the tiles that
// share an L2 also share A and B panels.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
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

// global -> LDS without passing through registers.  Written as inline assembly on purpose: the
// compiler's wait-count insertion treats every LDS read as possibly aliasing an outstanding
// global_load_lds and would drain all loads (vmcnt(0)) before each fragment read, which defeats the
// prefetch ring; the kernel waits explicitly for the one tile it is about to read instead.
// LDS destination = lds_base (wave-uniform, via M0) + lane * size.  The "memory" clobber tells the compiler what it cannot
// see in the statement: that it writes LDS, so no fragment read may be moved across it (costs nothing measurable).
// addressed as uniform 64-bit base (SGPR pair) + per-lane 32-bit byte offset: no 64-bit VGPR address math
__device__ __forceinline__ void load_lds_b128_s(const uint8_t* base, uint32_t lane_off, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(lds_base) : "memory");
}
// s_waitcnt immediate that waits for the vector-memory counter only
constexpr int vmcnt_imm(int n) { return 0x0f70 | (n & 0xf) | ((n >> 4) << 14); }
__device__ __forceinline__ void load_lds_b32(const uint8_t* gsrc, uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off" ::"v"(gsrc), "s"(lds_base) : "memory");
}

struct SubFrags {
    uint4 a[4], b[4];  // one K sub-step (64 values): four A tiles, four B tiles
};

// frag_off = byte offset of this lane's 16 bytes for the wanted sub-step within tile 0 of its operand
__device__ __forceinline__ void big_read_sub(const uint8_t* __restrict__ stage, int a_off, int b_off, SubFrags& f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f.a[i] = *reinterpret_cast<const uint4*>(stage + a_off + i * 32 * kRowBytes);
        f.b[i] = *reinterpret_cast<const uint4*>(stage + kBOff + b_off + i * 32 * kRowBytes);
    }
}

// SWAP = false: A rows become result rows.  SWAP = true: B's rows (n) are fed as the MFMA's first operand and
// A's rows (m) as its second, so a lane ends up with 4 consecutive n of one m (contiguous in row-major C),
// which the bf16 epilogue packs into 8-byte LDS writes.
template <int SUB, bool SWAP, bool ZERO = false>
__device__ __forceinline__ void big_mfma_sub(const SubFrags& f, const uint32_t (&sca)[4], const uint32_t (&scb)[4],
                                             v16f (&acc)[4][4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const v8i av = v8i{(int)f.a[i].x, (int)f.a[i].y, (int)f.a[i].z, (int)f.a[i].w, 0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const v8i bv = v8i{(int)f.b[j].x, (int)f.b[j].y, (int)f.b[j].z, (int)f.b[j].w, 0, 0, 0, 0};
            // ZERO: the tile's first product starts the accumulator from the constant 0 instead of reading it
            v16f cin;
            if constexpr (ZERO) {
#pragma unroll
                for (int e = 0; e < 16; ++e) cin[e] = 0.0f;
            } else {
                cin = acc[i][j];
            }
            if constexpr (SWAP)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, cin, 4, 4, SUB, (int)scb[j], SUB, (int)sca[i]);
            else
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, cin, 4, 4, SUB, (int)sca[i], SUB, (int)scb[j]);
        }
    }
}

// one MFMA, then one memory instruction of the given class, n times: keeps the matrix pipe fed while the
// wave issues its LDS / VMEM instructions
#define QM_SCHED_PAIR(mask, n)                                   \
    for (int _i = 0; _i < (n); ++_i) {                           \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);       \
        __builtin_amdgcn_sched_group_barrier((mask), 1, 0);      \
    }

// ---- two workgroups per CU: 256 x 128 tiles for short contractions -------------------------------------------------
// With a short K the tile boundary dominates: the 256 x 256 kernels spend about 7.5 k cycles per tile converting, staging
// and storing the result while no matrix instruction runs, against 1.3 k cycles per K step.  Here a workgroup owns a
// 256 x 128 tile with four waves of 128 x 64 (128 accumulator registers, at most 256 registers per wave), so a SIMD holds
// one wave of each of two workgroups: while one of them waits at its barrier, requests operands, or converts and stores
// its tile, the other's matrix instructions keep the pipe busy.  The price is 1.5 x the operand traffic per flop (LDS
// fragment reads and global -> LDS bytes), which is why long contractions stay on the 256 x 256 kernel.
// Three-stage ring per workgroup (3 x 25.5 KiB: codes of 256 + 128 rows and one scale dword per row and K step); the
// ring doubles as the epilogue's staging area, so nothing is prefetched across tiles -- the neighbour workgroup covers
// the gap.  Persistent: the grid is two workgroups per CU.  M, N multiples of 64, M >= 256, N >= 128, K % 128 == 0, or
// K % 128 == 64 with row-major operands (a final half step, see duo_issue).
constexpr int kDuoM = 256, kDuoN = 128, kDuoStages = 3;
constexpr int kDuoBOff = kDuoM * kRowBytes;                                   // 16 KiB of A codes
constexpr int kDuoSAOff = (kDuoM + kDuoN) * kRowBytes;                        // 24 KiB of codes
constexpr int kDuoSBOff = kDuoSAOff + kDuoM * 4;
constexpr int kDuoStageBytes = kDuoSBOff + kDuoN * 4;                         // 25.5 KiB
constexpr int kDuoSmemBytes = kDuoStages * kDuoStageBytes;                    // 76.5 KiB
constexpr int kDuoEpiPitch = 144;   // bytes per staged row of 64 bf16: 128 rows x 144 B = 18 KiB per wave
#ifndef QM_DUO_MAX_K
#define QM_DUO_MAX_K 768
#endif
constexpr int kDuoMaxK = QM_DUO_MAX_K;  // longest contraction served by this kernel
constexpr int kDuoLoads = 8;        // VMEM instructions per wave per K step: 4 (A) + 2 (B) + 2 (scales)
static_assert(4 * 128 * kDuoEpiPitch <= kDuoSmemBytes, "the epilogue stages through the operand ring");

struct DuoFrags {
    uint4 a[4], b[2];
};
struct DuoPlan {
    const uint8_t* a;   // uniform: this wave's 64 A rows of the tile, K step 0
    const uint8_t* b;   // uniform: this wave's 32 B rows
    const uint8_t* sa;  // this lane's A scale dword source at K step 0 (+ ks * 4 bytes)
    const uint8_t* sb;
    int64_t row16_bytes;
    uint32_t lane_codes_a, lane_codes_b;
    uint32_t half_codes_a, half_codes_b;  // the same for a final half step (K % 128 == 64): the row's last 32 bytes twice
    int kstep_a, kstep_b;
    uint32_t lds_a, lds_b, lds_sa, lds_sb;  // wave-uniform LDS addresses (stage 0)
};
// half: the step covers only 64 contraction indices (the last step of a K with K % 128 == 64, row-major operands).  Its
// lanes request the row's final two 16-byte pieces in place of all four, and the scale dword that ends with the row's last
// byte (two bytes early), so that no request leaves the row; the consumer shifts that dword down by 16 bits, which puts
// the two real scale bytes first and zeros (2^-127: products vanish) where the missing half of the step would be.
__device__ __forceinline__ void duo_issue(const DuoPlan& p, int stage, int ks, bool half) {
    const uint32_t off = (uint32_t)stage * kDuoStageBytes;
    const uint32_t la = half ? p.half_codes_a : p.lane_codes_a, lb = half ? p.half_codes_b : p.lane_codes_b;
#pragma unroll
    for (int j = 0; j < 4; ++j) load_lds_b128_s(p.a + j * p.row16_bytes + ks * p.kstep_a, la, p.lds_a + off + j * 1024);
#pragma unroll
    for (int j = 0; j < 2; ++j) load_lds_b128_s(p.b + j * p.row16_bytes + ks * p.kstep_b, lb, p.lds_b + off + j * 1024);
    const int sback = half ? 2 : 0;
    load_lds_b32(p.sa + ks * 4 - sback, p.lds_sa + off);
    load_lds_b32(p.sb + ks * 4 - sback, p.lds_sb + off);
}
__device__ __forceinline__ void duo_read_sub(const uint8_t* __restrict__ stage, int a_off, int b_off, DuoFrags& f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f.a[i] = *reinterpret_cast<const uint4*>(stage + a_off + i * 32 * kRowBytes);
#pragma unroll
    for (int j = 0; j < 2; ++j) f.b[j] = *reinterpret_cast<const uint4*>(stage + b_off + j * 32 * kRowBytes);
}
template <int SUB, bool SWAP, bool ZERO>
__device__ __forceinline__ void duo_mfma_sub(const DuoFrags& f, const uint32_t (&sca)[4], const uint32_t (&scb)[2], v16f (&acc)[4][2]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const v8i av = v8i{(int)f.a[i].x, (int)f.a[i].y, (int)f.a[i].z, (int)f.a[i].w, 0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const v8i bv = v8i{(int)f.b[j].x, (int)f.b[j].y, (int)f.b[j].z, (int)f.b[j].w, 0, 0, 0, 0};
            v16f cin;
            if constexpr (ZERO) {
#pragma unroll
                for (int e = 0; e < 16; ++e) cin[e] = 0.0f;
            } else {
                cin = acc[i][j];
            }
            if constexpr (SWAP)
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, cin, 4, 4, SUB, (int)scb[j], SUB, (int)sca[i]);
            else
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, cin, 4, 4, SUB, (int)sca[i], SUB, (int)scb[j]);
        }
    }
}

template <typename OutT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_mxfp4_tn_duo_kernel(
    const uint8_t* __restrict__ a_codes, const uint8_t* __restrict__ a_scales, const uint8_t* __restrict__ b_codes,
    const uint8_t* __restrict__ b_scales, int M, int N, int K, float alpha, OutT* __restrict__ c, int a_tiled, int b_tiled) {
    extern __shared__ uint32_t smem[];
    uint8_t* smem_bytes = reinterpret_cast<uint8_t*>(smem);
    const uint32_t smem_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t*)smem;
    constexpr bool SWAP = sizeof(OutT) == 2;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, half = lane >> 5;
    const int tiles_m = (M + kDuoM - 1) / kDuoM, tiles_n = (N + kDuoN - 1) / kDuoN, total = tiles_m * tiles_n;
    const int code_pitch = K / 2, groups = K / 32;
    const int nk = (K + kBK - 1) / kBK;
    const int half_step = (K % kBK) ? nk - 1 : -1;  // the K step that covers only 64 indices (K % 128 == 64), or none

    const int swz = (lrow >> 2) & 3;
    const int a_off0 = (wm * 128 + lrow) * kRowBytes + (((2 * half) ^ swz) * 16);
    const int a_off1 = (wm * 128 + lrow) * kRowBytes + (((2 * half + 1) ^ swz) * 16);
    const int b_off0 = kDuoBOff + (wn * 64 + lrow) * kRowBytes + (((2 * half) ^ swz) * 16);
    const int b_off1 = kDuoBOff + (wn * 64 + lrow) * kRowBytes + (((2 * half + 1) ^ swz) * 16);
    // scales in LDS: A dword p holds row (p >> 7) * 128 + (p & 3) * 32 + ((p >> 2) & 31), so one 16-byte read fetches the
    // scale dwords of a lane's four A tiles; B dword p holds row (p >> 6) * 64 + (p & 1) * 32 + ((p >> 1) & 31): one 8-byte read
    const int a_sc_off = kDuoSAOff + (wm * 32 + lrow) * 16;
    const int b_sc_off = kDuoSBOff + (wn * 32 + lrow) * 8;
    const int sh = 16 * half;

    DuoPlan plan;
    plan.row16_bytes = (int64_t)16 * code_pitch;
    {
        const int prow = lane >> 2;
        const int pcv = (lane & 3) ^ ((prow >> 2) & 3);
        const uint32_t rowmajor_off = (uint32_t)(prow * code_pitch + pcv * 16);
        const uint32_t tiled_off = (uint32_t)(prow * 64 + pcv * 16);
        plan.lane_codes_a = a_tiled ? tiled_off : rowmajor_off;
        plan.lane_codes_b = b_tiled ? tiled_off : rowmajor_off;
        // a half step exists for row-major operands only: pieces 2 and 3 of the step lie beyond the row, their LDS slots
        // receive pieces 0 and 1 again (and zero scales)
        plan.half_codes_a = plan.half_codes_b = (uint32_t)(prow * code_pitch + (pcv & 1) * 16);
        plan.kstep_a = a_tiled ? 1024 : kRowBytes;
        plan.kstep_b = b_tiled ? 1024 : kRowBytes;
        plan.lds_a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_base + wave * 4096));
        plan.lds_b = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_base + kDuoBOff + wave * 2048));
        plan.lds_sa = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_base + kDuoSAOff + wave * 256));
        // 128 B scale dwords: waves 2 and 3 repeat the requests of waves 0 and 1 (same bytes to the same place), which
        // keeps every wave's count of outstanding loads the same
        plan.lds_sb = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_base + kDuoSBOff + (wave & 1) * 256));
    }
    // operand rows behind the scale dwords this lane requests
    const int pa = wave * 64 + lane, pb = (wave & 1) * 64 + lane;
    const int srow_a = (pa >> 7) * 128 + (pa & 3) * 32 + ((pa >> 2) & 31);
    const int srow_b = (pb >> 6) * 64 + (pb & 1) * 32 + ((pb >> 1) & 31);

    for (int t = (int)blockIdx.x; t < total; t += (int)gridDim.x) {
        int tm, tn;
        tile_of_block(t, tiles_m, tiles_n, tm, tn);
        const int64_t m0 = (int64_t)tm * kDuoM, n0 = (int64_t)tn * kDuoN;
        {
            // M and N are multiples of 64 (32 for a wave's share of B): a wave's share of a panel lies inside the matrix or
            // outside it as a whole; an outside share reads the matrix's last rows instead (its products are dropped below)
            int64_t ma = m0 + wave * 64, nb = n0 + wave * 32;
            ma = ma < M ? ma : (int64_t)M - 64;
            nb = nb < N ? nb : (int64_t)N - 32;
            plan.a = a_codes + ma * code_pitch;
            plan.b = b_codes + nb * code_pitch;
            plan.sa = a_scales + (m0 + srow_a < M ? m0 + srow_a : (int64_t)M - 1) * groups;
            plan.sb = b_scales + (n0 + srow_b < N ? n0 + srow_b : (int64_t)N - 1) * groups;
        }
        const int rows_valid = (int)(M - m0) - wm * 128, cols_valid = (int)(N - n0) - wn * 64;

        const auto issue = [&](int stage, int ks) { duo_issue(plan, stage, ks, ks == half_step); };
        // the scale dwords of a half step arrive two bytes early (see duo_issue).  Without a branch: a K step is one basic
        // block, which is what holds its instruction order in place.
        const auto settle_scales = [&](uint4& a, uint2& b, int ks) {
            const uint32_t down = ks == half_step ? 16u : 0u;
            a.x >>= down; a.y >>= down; a.z >>= down; a.w >>= down;
            b.x >>= down; b.y >>= down;
        };
        issue(0, 0);
        issue(1, nk > 1 ? 1 : 0);
        issue(2, nk > 2 ? 2 : nk - 1);
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(2 * kDuoLoads));  // step 0 is in; steps 1, 2 may be pending
        __syncthreads();
        DuoFrags f0, f1;
        uint4 sa4 = *reinterpret_cast<const uint4*>(smem_bytes + a_sc_off);
        uint2 sb2 = *reinterpret_cast<const uint2*>(smem_bytes + b_sc_off);
        settle_scales(sa4, sb2, 0);
        duo_read_sub(smem_bytes, a_off0, b_off0, f0);

        v16f acc[4][2];
        int stage = 0;
        // one K step: `stage` is the ring slot it consumes and then refills with step s + 3
        auto step = [&](auto first_tag, int s) {
            constexpr bool FIRST = decltype(first_tag)::value;
            const int nstage = stage == kDuoStages - 1 ? 0 : stage + 1;
            const uint8_t* cur = smem_bytes + stage * kDuoStageBytes;
            const uint8_t* nxt = smem_bytes + nstage * kDuoStageBytes;
            const uint32_t sca[4] = {__builtin_amdgcn_ubfe(sa4.x, (uint32_t)sh, 16u), __builtin_amdgcn_ubfe(sa4.y, (uint32_t)sh, 16u),
                                     __builtin_amdgcn_ubfe(sa4.z, (uint32_t)sh, 16u), __builtin_amdgcn_ubfe(sa4.w, (uint32_t)sh, 16u)};
            const uint32_t scb[2] = {__builtin_amdgcn_ubfe(sb2.x, (uint32_t)sh, 16u), __builtin_amdgcn_ubfe(sb2.y, (uint32_t)sh, 16u)};
            duo_read_sub(cur, a_off1, b_off1, f1);
            duo_mfma_sub<0, SWAP, FIRST>(f0, sca, scb, acc);
            QM_SCHED_PAIR(0x100, 6)
            __builtin_amdgcn_sched_barrier(0);
            // younger than the loads of step s + 1: those of step s + 2
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(kDuoLoads));
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            // past the end: a repeat nobody reads keeps the counts of outstanding loads uniform
            issue(stage, s + 3 < nk ? s + 3 : nk - 1);
            sa4 = *reinterpret_cast<const uint4*>(nxt + a_sc_off);
            sb2 = *reinterpret_cast<const uint2*>(nxt + b_sc_off);
            settle_scales(sa4, sb2, s + 1);
            duo_read_sub(nxt, a_off0, b_off0, f0);
            duo_mfma_sub<1, SWAP, false>(f1, sca, scb, acc);
            QM_SCHED_PAIR(0x100, 6)
            __builtin_amdgcn_sched_barrier(0);
            stage = nstage;
        };
        step(std::true_type{}, 0);
        for (int ks = 1; ks < nk; ++ks) step(std::false_type{}, ks);
        // every request has landed and every wave has read its last fragments: the ring becomes the staging area
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        __syncthreads();
        if constexpr (SWAP) {
            uint8_t* region = smem_bytes + wave * (128 * kDuoEpiPitch);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        const v16f& v = acc[i][j];
                        const v2bf p0 = __builtin_convertvector(v2f{v[4 * b] * alpha, v[4 * b + 1] * alpha}, v2bf);
                        const v2bf p1 = __builtin_convertvector(v2f{v[4 * b + 2] * alpha, v[4 * b + 3] * alpha}, v2bf);
                        *reinterpret_cast<uint2*>(region + (i * 32 + lrow) * kDuoEpiPitch + (j * 32 + 8 * b + 4 * half) * 2) =
                            make_uint2(__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1));
                    }
            // the region is private to the wave; LDS operations of one wave complete in order
            const int chunk = lane & 7, rsub = lane >> 3;
            uint8_t* out = reinterpret_cast<uint8_t*>(reinterpret_cast<uint16_t*>(c) + (m0 + wm * 128 + rsub) * N + n0 + wn * 64) + chunk * 16;
            const int64_t pitch8 = (int64_t)N * 16;  // eight rows of bf16
            if (cols_valid > 0) {
#pragma unroll
                for (int r8 = 0; r8 < 16; ++r8) {
                    const uint4 v = *reinterpret_cast<const uint4*>(region + (r8 * 8 + rsub) * kDuoEpiPitch + chunk * 16);
                    typedef uint32_t u4v __attribute__((ext_vector_type(4)));
                    if (r8 * 8 < rows_valid) __builtin_nontemporal_store(u4v{v.x, v.y, v.z, v.w}, reinterpret_cast<u4v*>(out + r8 * pitch8));
                }
            }
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    if (i * 32 < rows_valid && j * 32 < cols_valid)
                        store_tile<OutT>(acc[i][j], alpha, c, m0 + wm * 128 + i * 32, n0 + wn * 64 + j * 32 + lrow, N, half);
        }
        __syncthreads();  // the staging area is the next tile's ring
    }
}

// ---- persistent variant: scales travel in blocks of four K steps ------------------------------------
// Fetching one scale dword per row per K step costs as many L2 requests as the codes themselves (each
// row's 4 bytes sit in a different cache line).  Here a wave-load brings 16 bytes per row = the scales of
// four K steps, into a small double-buffered LDS area behind the four code stages; a lane reads the
// scale vectors of its eight tile rows once per block and keeps them in registers.
constexpr int kCodeStageBytes = (kBigM + kBigN) * kRowBytes;            // 32 KiB
constexpr int kScaleAreaOff = kStages * kCodeStageBytes;                // 128 KiB
constexpr int kScaleBufBytes = (kBigM + kBigN) * 16;                    // 8 KiB per block of four K steps
constexpr int kEpiAreaOff = kScaleAreaOff + 2 * kScaleBufBytes;     // 144 KiB
constexpr int kEpiWaveBytes = 4096;                                  // 32 rows x 64 bf16 per wave
constexpr int kBig4SmemBytes = kEpiAreaOff + 4 * kEpiWaveBytes;      // 160 KiB

struct Big4Plan {
    const uint8_t* a;   // uniform: first code byte of this tile's A panel (row m0, K step 0)
    const uint8_t* b;
    const uint8_t* sa;  // uniform: first scale byte of this tile's A panel
    const uint8_t* sb;
    int64_t row16_bytes;    // 16 rows of codes
    uint32_t lane_codes_a;  // this lane's byte offset inside a wave-load's source: row lane/4 + swizzled 16-byte column of a
    uint32_t lane_codes_b;  //   row-major panel, or the same pick inside the 1 KiB tile of a tiled one
    int kstep_a, kstep_b;   // bytes from one K step to the next: 64 row-major, 1024 tiled
    uint32_t voff_a[4];     // lane_codes_a + i * (row16_bytes - 1024): wave-load i of a K step, issued with instruction
    uint32_t voff_b[4];     //   offset i * 1024, which moves its LDS destination by as much (and the source back in place)
    uint32_t lane_scales;   // this lane's byte offset inside a panel's scales: row wave*64 + lane
    uint32_t lds_codes;     // wave-uniform LDS address of this wave's first A wave-load in stage 0
    uint32_t lds_scales;    // wave-uniform LDS address of this wave's A scale wave-load in buffer 0
};

__device__ __forceinline__ void big4_issue_codes(const Big4Plan& p, int stage, int ks) {
    const uint32_t base = p.lds_codes + stage * kCodeStageBytes;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        load_lds_b128_s(p.a + j * p.row16_bytes + ks * p.kstep_a, p.lane_codes_a, base + j * 1024);
        load_lds_b128_s(p.b + j * p.row16_bytes + ks * p.kstep_b, p.lane_codes_b, base + kBOff + j * 1024);
    }
}
// soff: byte offset, within a row's scales, of the 16 bytes (four K steps) to request
__device__ __forceinline__ void big4_issue_scales(const Big4Plan& p, int soff, int buf) {
    const uint32_t base = p.lds_scales + buf * kScaleBufBytes;
    load_lds_b128_s(p.sa + soff, p.lane_scales, base);
    load_lds_b128_s(p.sb + soff, p.lane_scales, base + kBigM * 16);
}

// The LDS destination of a global->LDS load is M0 + the instruction's offset + lane * 16, and the same offset is added
// to the source address: with the lane offsets of Big4Plan::voff_* one M0 value serves the four wave-loads of an
// operand, and the loads themselves are single instructions between the MFMAs (every instruction a wave issues costs
// it four to five cycles, and a K step has only 32 cycles per MFMA to hide them in).
__device__ __forceinline__ void set_lds_dma_base(uint32_t lds_base) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0" ::"s"(lds_base));
}
template <int I>
__device__ __forceinline__ void load_lds_b128_m0(const uint8_t* base, uint32_t lane_off) {
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" ::"v"(lane_off), "s"(base), "i"(I * 1024) : "memory");
}

struct ScaleRegs {
    uint4 a[4], b[4];  // per tile: the row's scale dwords of the block's four K steps
};
__device__ __forceinline__ void big4_read_scales(const uint8_t* __restrict__ sbuf, int a_off, int b_off, ScaleRegs& r) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        r.a[i] = *reinterpret_cast<const uint4*>(sbuf + a_off + i * 32 * 16);
        r.b[i] = *reinterpret_cast<const uint4*>(sbuf + kBigM * 16 + b_off + i * 32 * 16);
    }
}
template <int Q>
__device__ __forceinline__ uint32_t pick(const uint4& v) {
    return Q == 0 ? v.x : (Q == 1 ? v.y : (Q == 2 ? v.z : v.w));
}


struct Big4State {
    SubFrags f0, f1;
    ScaleRegs sr;
};

// One K step of the flat (tile, K step) stream; the step's index in its tile is congruent to Q mod 4, so
// the ring stage it consumes is Q.  `lks` is the K step (of the tile `plan` points at) whose codes it
// requests into the stage it has just freed, `soff` (Q = 0 only) the byte offset of the scale block it requests;
// `sw` = 16, or 0 for a step whose scale bytes are to read as zero (2^-127: its products vanish); `par` selects the
// scale buffer the current block lives in.
template <int Q, bool SWAP, bool FIRST = false, int EXTRA = 0>
__device__ __forceinline__ void big4_step(const Big4Plan& plan, uint8_t* smem_bytes, int lks, int soff, int sw, int par, int a_off0,
                                          int a_off1, int b_off0, int b_off1, int a_sc_off, int b_sc_off, int sh,
                                          Big4State& st, v16f (&acc)[4][4]) {
    const uint8_t* cur = smem_bytes + Q * kCodeStageBytes;
    const uint8_t* nxt = smem_bytes + ((Q + 1) & 3) * kCodeStageBytes;
    // the lane half's two scale bytes of this step: bits [sh, sh + 16) of the row's dword; sw = 0 mutes the step
    const auto two = [&](const uint4& v) { return __builtin_amdgcn_ubfe(pick<Q>(v), (uint32_t)sh, (uint32_t)sw); };
    const uint32_t sca[4] = {two(st.sr.a[0]), two(st.sr.a[1]), two(st.sr.a[2]), two(st.sr.a[3])};
    const uint32_t scb[4] = {two(st.sr.b[0]), two(st.sr.b[1]), two(st.sr.b[2]), two(st.sr.b[3])};
    big_read_sub(cur, a_off1, b_off1, st.f1);
    big_mfma_sub<0, SWAP, FIRST>(st.f0, sca, scb, acc);
    QM_SCHED_PAIR(0x100, 8)
    __builtin_amdgcn_sched_barrier(0);
    // loads younger than the codes of the next step: the codes of the two steps after it (16) and, for Q = 1, 2,
    // the two scale loads issued since; for Q = 3 the scale block read below is older than those and must be in
    // EXTRA: requests of another kind issued since the awaited stage's (the fused epilogue's mask words, which a tile
    // requests at its first K step and which may stay pending through its first three)
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(((Q == 1 || Q == 2) ? 18 : 16) + EXTRA));
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (Q == 3) big4_read_scales(smem_bytes + kScaleAreaOff + (par ^ 1) * kScaleBufBytes, a_sc_off, b_sc_off, st.sr);
    // one quarter of the step's requests and fragment reads per four MFMAs (same issue order as the clumped form)
    {
        const uint32_t base = plan.lds_codes + Q * kCodeStageBytes;
        if constexpr (Q == 3) __builtin_amdgcn_sched_barrier(0);
        const uint8_t* src_a = plan.a + lks * plan.kstep_a;  // uniform: this wave's panel rows, K step lks
        const uint8_t* src_b = plan.b + lks * plan.kstep_b;
        set_lds_dma_base(base);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const v8i av = v8i{(int)st.f1.a[i].x, (int)st.f1.a[i].y, (int)st.f1.a[i].z, (int)st.f1.a[i].w, 0, 0, 0, 0};
            const auto products = [&](int j0, int j1) {
#pragma unroll
                for (int j = j0; j < j1; ++j) {
                    const v8i bv = v8i{(int)st.f1.b[j].x, (int)st.f1.b[j].y, (int)st.f1.b[j].z, (int)st.f1.b[j].w, 0, 0, 0, 0};
                    if constexpr (SWAP)
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bv, av, acc[i][j], 4, 4, 1, (int)scb[j], 1, (int)sca[i]);
                    else
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc[i][j], 4, 4, 1, (int)sca[i], 1, (int)scb[j]);
                }
            };
            // per four MFMAs: two fragment reads of the next stage and two of the step's eight wave-loads (A's four,
            // then B's four behind a second M0 value)
            st.f0.a[i] = *reinterpret_cast<const uint4*>(nxt + a_off0 + i * 32 * kRowBytes);
            if (i == 0) load_lds_b128_m0<0>(src_a, plan.voff_a[0]);
            if (i == 1) load_lds_b128_m0<2>(src_a, plan.voff_a[2]);
            if (i == 2) { set_lds_dma_base(base + kBOff); load_lds_b128_m0<0>(src_b, plan.voff_b[0]); }
            if (i == 3) load_lds_b128_m0<2>(src_b, plan.voff_b[2]);
            st.f0.b[i] = *reinterpret_cast<const uint4*>(nxt + kBOff + b_off0 + i * 32 * kRowBytes);
            if (i == 0) load_lds_b128_m0<1>(src_a, plan.voff_a[1]);
            if (i == 1) load_lds_b128_m0<3>(src_a, plan.voff_a[3]);
            if (i == 2) load_lds_b128_m0<1>(src_b, plan.voff_b[1]);
            if (i == 3) load_lds_b128_m0<3>(src_b, plan.voff_b[3]);
            if constexpr (Q == 0) {
                if (i == 3) big4_issue_scales(plan, soff, par ^ 1);
            }
            products(0, 4);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// bf16 epilogue (operand roles swapped: a lane's accumulator quads run along n).  Eight passes of 32 rows x 64
// columns per wave through a private 4 KiB LDS stage outside the operand ring, so the next tile's operands
// keep streaming in underneath; 16-byte chunks are XOR-swizzled by row so that writes and reads spread over
// all banks.
// ROT: the masked inverse Hadamard rotation of the layer's backward pass (groups of 32 along n) applied to the tile before it
// is stored: out[m][n'] = c * sum_n (bf16(alpha * acc[m][n]) * keep[m][n]) * S[n'][n] * sign[n], S the 32 x 32 Sylvester
// matrix.  With the operand roles swapped a lane holds 16 of a group's 32 n for one m, which is the layout the bf16
// matrix instruction reads its second operand in (k along the registers, column = lane % 32); its first operand is the
// +-1 matrix, rebuilt per tile from the sign word.  The sums are fp32 sums of bf16 values in the instruction's order
// (the stand-alone kernel adds them as a butterfly), the factor c and the final rounding are the same.
struct RotEpilogue {
    const uint8_t* mask;  // [M][N / 8] clip-mask bits, bit n % 8 of byte n / 8
    uint32_t signs;       // bit n: column n of the Hadamard block negated
    float c;              // 32^-1/2, rounded to the scale dtype
};
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <bool ROT = false>
__device__ __forceinline__ void big4_epilogue_bf16(v16f (&acc)[4][4], float alpha, uint16_t* __restrict__ c, int64_t m0,
                                                   int64_t n0, int64_t N, int wm, int wn, int wave, int lane_in,
                                                   uint8_t* smem_bytes, int rows_valid, int cols_valid,
                                                   [[maybe_unused]] const RotEpilogue& rot, [[maybe_unused]] const u32x4 (&keep)[4],
                                                   [[maybe_unused]] bool keep_shifted) {
    // The opaque copy keeps the address arithmetic below inside the (rarely executed) epilogue instead of being
    // hoisted out of the K loop, where it would hold dozens of registers across the MFMA schedule.
    // the lane index straight from the hardware, so that no copy of it has to stay alive through the K loop
    (void)lane_in;
    int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    asm volatile("" : "+v"(lane));
    const int lrow = lane & 31, half = lane >> 5;
    uint8_t* region = smem_bytes + kEpiAreaOff + wave * kEpiWaveBytes;
    const int chunk = lane & 7, rsub = lane >> 3;
    uint8_t* wr = region + lrow * 128 + half * 8;
    const int wsw = (lrow & 7) * 16;
    const uint8_t* rd = region + rsub * 128 + ((chunk ^ rsub) * 16);  // rows rsub + 8k share rsub's swizzle
    const int64_t pitch8 = N * 16;                                   // eight rows of bf16
    uint8_t* out = reinterpret_cast<uint8_t*>(c + (m0 + wm * 128 + rsub) * N + n0 + wn * 128) + chunk * 16;
    // ROT: `keep[i]` holds the four mask words of the lane's row in block row i (one per 32 x 32 block: its group of 32 n),
    // requested at the tile's first K step.  The +-1 matrix: lane (n' = lane % 32, half h) holds, for instruction q,
    // S[n'][n] sign[n] at n = 8 (2 q + rho) + 4 h + e
    [[maybe_unused]] v8bf hmat[2];
    // a factor c that bf16 holds exactly (the bf16 scale dtype) rides in the matrix entries: the products stay exact in fp32
    // and the multiplication after the sums falls away
    [[maybe_unused]] const bool c_in_matrix = ROT && (f2u(rot.c) & 0xffffu) == 0u;
    if constexpr (ROT) {
        const uint32_t one = c_in_matrix ? f2u(rot.c) >> 16 : 0x3f80u;
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            uint32_t w[4];
#pragma unroll
            for (int pr = 0; pr < 4; ++pr) {   // pair pr: rho = pr / 2, e = 2 (pr % 2), +1
                uint32_t bits = 0u;
#pragma unroll
                for (int k = 0; k < 2; ++k) {
                    const int n = 8 * (2 * q + pr / 2) + 4 * half + 2 * (pr & 1) + k;
                    const uint32_t neg = ((uint32_t)__builtin_popcount((uint32_t)(lrow & n)) ^ (rot.signs >> n)) & 1u;
                    bits |= (one | (neg << 15)) << (16 * k);
                }
                w[pr] = bits;
            }
            hmat[q] = __builtin_bit_cast(v8bf, u32x4{w[0], w[1], w[2], w[3]});
        }
    }
    acc_settle();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int jp = 0; jp < 2; ++jp) {
            if (i * 32 >= rows_valid || jp * 64 >= cols_valid) continue;  // uniform: this pass lies outside the matrix
            if constexpr (!ROT) {
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
#pragma unroll
                    for (int b = 0; b < 4; ++b) {
                        const v16f& t = acc[i][2 * jp + jj];
                        const float t0 = acc_read(t[4 * b]), t1 = acc_read(t[4 * b + 1]), t2 = acc_read(t[4 * b + 2]), t3 = acc_read(t[4 * b + 3]);
                        const v2bf p0 = __builtin_convertvector(v2f{t0 * alpha, t1 * alpha}, v2bf);
                        const v2bf p1 = __builtin_convertvector(v2f{t2 * alpha, t3 * alpha}, v2bf);
                        *reinterpret_cast<uint2*>(wr + (((jj * 4 + b) * 16) ^ wsw)) =
                            make_uint2(__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1));
                    }
                }
            } else {
                // Both blocks of the pass go through the matrix pipe before either result is read: the second block's
                // conversion and masking run while the first block's instructions are in flight (the opaque copies below
                // keep the read-out of the results behind both blocks' matrix instructions).  Per tile 15.9 k -> 14.7 k cycles.
                v16f r[2];
#pragma unroll
                for (int jj = 0; jj < 2; ++jj) {
                    const v16f& t = acc[i][2 * jp + jj];
                    // the block rounded to bf16 and masked: register pair 2 b + k holds n = 8 b + 4 half + 2 k, + 1
                    // the block's mask word: word j of the row's four, or word j + 2 where the wave requested the row's last
                    // 16 bytes (its columns hang over the edge of N; blocks 2 and 3 are then outside and skipped)
                    const uint32_t kword = keep_shifted ? keep[i][(2 * jp + jj + 2) & 3] : keep[i][2 * jp + jj];
                    const uint32_t kw = kword >> (4 * half);
                    uint32_t pk[8];
#pragma unroll
                    for (int b = 0; b < 4; ++b)
#pragma unroll
                        for (int k = 0; k < 2; ++k) {
                            const float t0 = acc_read(t[4 * b + 2 * k]), t1 = acc_read(t[4 * b + 2 * k + 1]);
                            const uint32_t p = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{t0 * alpha, t1 * alpha}, v2bf));
                            const uint32_t lo = (uint32_t)__builtin_amdgcn_sbfe((int)kw, 8 * b + 2 * k, 1);       // 0 or ~0
                            const uint32_t hi = (uint32_t)__builtin_amdgcn_sbfe((int)kw, 8 * b + 2 * k + 1, 1);
                            pk[2 * b + k] = p & ((lo & 0xffffu) | (hi & 0xffff0000u));
                        }
                    v16f z;
#pragma unroll
                    for (int e = 0; e < 16; ++e) z[e] = 0.0f;
                    z = __builtin_amdgcn_mfma_f32_32x32x16_bf16(hmat[0], __builtin_bit_cast(v8bf, u32x4{pk[0], pk[1], pk[2], pk[3]}), z, 0, 0, 0);
                    r[jj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(hmat[1], __builtin_bit_cast(v8bf, u32x4{pk[4], pk[5], pk[6], pk[7]}), z, 0, 0, 0);
                }
                const auto emit = [&](auto scaled) {
#pragma unroll
                    for (int jj = 0; jj < 2; ++jj) {
                        asm volatile("" : "+v"(r[jj]));
#pragma unroll
                        for (int b = 0; b < 4; ++b) {
                            float q[4];
#pragma unroll
                            for (int e = 0; e < 4; ++e) q[e] = decltype(scaled)::value ? r[jj][4 * b + e] * rot.c : r[jj][4 * b + e];
                            const v2bf p0 = __builtin_convertvector(v2f{q[0], q[1]}, v2bf);
                            const v2bf p1 = __builtin_convertvector(v2f{q[2], q[3]}, v2bf);
                            *reinterpret_cast<uint2*>(wr + (((jj * 4 + b) * 16) ^ wsw)) =
                                make_uint2(__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1));
                        }
                    }
                };
                if (c_in_matrix) emit(std::false_type{});
                else emit(std::true_type{});
            }
            // the region is private to the wave; LDS operations of one wave complete in order
#pragma unroll
            for (int r8 = 0; r8 < 4; ++r8) {
                const uint4 v = *reinterpret_cast<const uint4*>(rd + r8 * 1024);
                // streaming store: the tile is not read again by this kernel, and keeping it out of the L2 leaves the
                // operand panels there (measured: -1.3 % on the product alone, -3 % on the whole layer step)
                typedef uint32_t u4v __attribute__((ext_vector_type(4)));
                __builtin_nontemporal_store(u4v{v.x, v.y, v.z, v.w}, reinterpret_cast<u4v*>(out + r8 * pitch8 + jp * 128));
            }
            // keeps the passes apart: a scheduler that reads many passes' accumulators into vector registers ahead of time
            // pushes the K loop's live values out to scratch memory, and their reloads wait for every operand load in flight
            __builtin_amdgcn_sched_barrier(0);
        }
        out += 4 * pitch8;
    }
}

// Measurement aid (the STAMP instantiation of the kernel below): the shader clock at a workgroup's entry, at the start of
// its tile loop, and after every tile's K loop and epilogue, kPhaseStamps values per workgroup at the kernel's `stamps`
// argument (which the production instantiation never reads).
constexpr int kPhaseStamps = 32;  // entry, loop start, then (K loop end, epilogue end) of up to 15 tiles
__device__ __forceinline__ unsigned long long shader_clock() {
    unsigned long long t;
    // the counter arrives like a scalar load: without the wait the registers it lands in may be reused before it does
    asm volatile("s_memtime %0\n\ts_waitcnt lgkmcnt(0)" : "=s"(t));
    return t;
}

// Persistent: the grid is one workgroup per CU (or fewer); each workgroup walks tiles bid, bid + grid, ... as one
// flat stream of K steps.  The loads that refill a freed ring stage simply continue into the next tile, so the
// pipeline never drains between tiles and the epilogue runs while the next tile's first four stages arrive.
template <typename OutT, bool STAMP = false, bool ROT = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void gemm_mxfp4_tn_big4_kernel(
    const uint8_t* __restrict__ a_codes, const uint8_t* __restrict__ a_scales, const uint8_t* __restrict__ b_codes,
    const uint8_t* __restrict__ b_scales, int M, int N, int K, float alpha, OutT* __restrict__ c, int a_tiled,
    int b_tiled, int splits, int late, [[maybe_unused]] unsigned long long* __restrict__ stamps,
    [[maybe_unused]] RotEpilogue rot = RotEpilogue{}) {
    static_assert(!ROT || sizeof(OutT) == 2, "the fused inverse rotation is part of the bf16 epilogue");
    extern __shared__ uint32_t smem[];
    uint8_t* smem_bytes = reinterpret_cast<uint8_t*>(smem);
    const uint32_t smem_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint32_t*)smem;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    [[maybe_unused]] int stamps_taken = 0;
    const auto stamp = [&]() {
        if constexpr (STAMP) {
            const unsigned long long now = shader_clock();
            if (tid == 0 && stamps_taken < kPhaseStamps) stamps[(size_t)blockIdx.x * kPhaseStamps + stamps_taken] = now;
            ++stamps_taken;
        }
    };
    stamp();
    // wave-uniform by construction; saying so keeps everything derived from it (tile corners, edge tests, the epilogue's
    // base addresses) in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int lrow = lane & 31, half = lane >> 5;
    const int tiles_m = (M + kBigM - 1) / kBigM, tiles_n = (N + kBigN - 1) / kBigN, total = tiles_m * tiles_n;
    const int code_pitch = K / 2, groups = K / 32;
    // Split K: a work item is (tile, K range); with splits > 1 (fp32 instantiation only) item (t, s) covers K steps
    // [s * nk, (s + 1) * nk) and stores its partial sums, unscaled, into slab s of c = [splits][M][N].
    // K steps per work item.  The pipeline walks blocks of four steps.  When K is not a multiple of 512 (one work item
    // then) the last block covers the row's final four steps, and those of them that the block before has already
    // added are muted: their scale bytes read as zero (2^-127 each), so every product is below the smallest fp32
    // denormal and adds an exact zero.  No request leaves the operand's rows.
    const int nk_real = K / kBK / splits;
    const int nk = (nk_real + 3) & ~3;
    const int muted = nk - nk_real;  // steps of the last block that repeat the block before (0: K steps in whole blocks)
    const int total_items = total * splits;
    const int stride = (int)gridDim.x;

    const int swz = (lrow >> 2) & 3;
    const int a_off0 = (wm * 128 + lrow) * kRowBytes + (((2 * half) ^ swz) * 16);
    const int a_off1 = (wm * 128 + lrow) * kRowBytes + (((2 * half + 1) ^ swz) * 16);
    const int b_off0 = (wn * 128 + lrow) * kRowBytes + (((2 * half) ^ swz) * 16);
    const int b_off1 = (wn * 128 + lrow) * kRowBytes + (((2 * half + 1) ^ swz) * 16);
    const int a_sc_off = (wm * 128 + lrow) * 16, b_sc_off = (wn * 128 + lrow) * 16;
    const int sh = 16 * half;

    Big4Plan plan;
    plan.row16_bytes = (int64_t)16 * code_pitch;
    plan.lds_codes = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_base + wave * 4096));
    plan.lds_scales = (uint32_t)__builtin_amdgcn_readfirstlane((int)(smem_base + kScaleAreaOff + wave * 1024));
    {
        const int prow = lane >> 2;  // the wave's 64-row offset is folded into the uniform part below
        const int pcv = (lane & 3) ^ ((prow >> 2) & 3);
        const uint32_t rowmajor_off = (uint32_t)(prow * code_pitch + pcv * 16);
        const uint32_t tiled_off = (uint32_t)(prow * 64 + pcv * 16);  // same (row, swizzled slot) pick inside the 1 KiB tile
        plan.lane_codes_a = a_tiled ? tiled_off : rowmajor_off;
        plan.lane_codes_b = b_tiled ? tiled_off : rowmajor_off;
        plan.kstep_a = a_tiled ? 1024 : kRowBytes;
        plan.kstep_b = b_tiled ? 1024 : kRowBytes;
        plan.lane_scales = (uint32_t)(lane * groups);
        const uint32_t step16 = (uint32_t)plan.row16_bytes - 1024u;  // 16 rows are 8 K bytes in either layout, K >= 512
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            plan.voff_a[i] = plan.lane_codes_a + (uint32_t)i * step16;
            plan.voff_b[i] = plan.lane_codes_b + (uint32_t)i * step16;
        }
    }
    const int wave_u = wave;
    int load_tm, load_tn, load_split;  // work item the load stream is in
    auto plan_tile = [&](int item) {
        const int t = item / splits;
        load_split = item - t * splits;
        tile_of_block(t, tiles_m, tiles_n, load_tm, load_tn);
        // M and N are multiples of 64: a wave's 64-row share of a panel is inside the matrix or outside it as a whole;
        // an outside share reads the matrix's last 64 rows instead (its products are dropped by the epilogue)
        int64_t m0 = (int64_t)load_tm * kBigM + wave_u * 64, n0 = (int64_t)load_tn * kBigN + wave_u * 64;
        m0 = m0 < M ? m0 : (int64_t)M - 64;
        n0 = n0 < N ? n0 : (int64_t)N - 64;
        const int64_t k0 = (int64_t)load_split * nk_real;  // first K step of the item
        plan.a = a_codes + m0 * code_pitch + k0 * plan.kstep_a;
        plan.b = b_codes + n0 * code_pitch + k0 * plan.kstep_b;
        plan.sa = a_scales + m0 * groups + k0 * 4;
        plan.sb = b_scales + n0 * groups + k0 * 4;
    };

    // Short contractions: every other group of eight workgroups (one per XCD) starts `late` x 1024 cycles late -- about the
    // length of an epilogue -- so that half of an XCD's CUs convert and store their tiles while the other half multiply.
    // Left alone the CUs can fall into step, and then every tile boundary is a burst of 33 MB of stores during which no CU
    // multiplies; which of the two states a launch settles in differs from chip to chip and from run to run (measured at
    // 32768 x 1536 x 1536: 53-57 us in step, 45-46 us out of step; with the late start always the latter).
    if (((int)blockIdx.x >> 3) & 1)
        for (int i = 0; i < late; ++i) __builtin_amdgcn_s_sleep(16);
    plan_tile((int)blockIdx.x);
    big4_issue_scales(plan, 0, 0);  // K >= 512: the first block is a whole one
    big4_issue_codes(plan, 0, 0);
    big4_issue_codes(plan, 1, 1);
    big4_issue_codes(plan, 2, 2);
    big4_issue_codes(plan, 3, 3);

    // scale block 0 and code stage 0 must be in; stages 1..3 (24 loads, the youngest) may be pending
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(24));
    __syncthreads();
    Big4State st;
    big4_read_scales(smem_bytes + kScaleAreaOff, a_sc_off, b_sc_off, st.sr);
    big_read_sub(smem_bytes, a_off0, b_off0, st.f0);

    int par = 0;
    stamp();
    for (int t = (int)blockIdx.x; t < total_items; t += stride) {
        v16f acc[4][4];
        const int64_t m0 = (int64_t)load_tm * kBigM, n0 = (int64_t)load_tn * kBigN;  // the load stream is still in item t
        const int cur_split = load_split;
        const int rows_valid = (int)(M - m0) - wm * 128, cols_valid = (int)(N - n0) - wn * 128;
        // One block of four K steps.  The load stream is four K steps ahead and rolls over into the next tile;
        // after the last tile it re-requests the current steps (never consumed), which keeps the outstanding-load
        // counts uniform.  FIRST: the tile's first products overwrite the accumulators instead of adding to them.
        // the fused epilogue's mask words: one per 32 x 32 block of the lane's row, requested here -- ahead of the tile's
        // first K step, so that the K loop hides their latency -- into registers the epilogue reads.  A row's four words
        // (the wave's 128 columns) are 16 contiguous bytes: one request per block row.  A wave whose columns hang over the
        // edge of N by half requests the row's last 16 bytes (its own two words come second there); rows below M and
        // waves wholly outside read the matrix's last row / columns and store nothing.
        // Nothing may read these registers before the epilogue (the data is in flight): the words are picked there.
        [[maybe_unused]] u32x4 keep[4];
        [[maybe_unused]] bool keep_shifted = false;
        if constexpr (ROT) {
            const int64_t mask_pitch = N / 8;
            int64_t ncol = n0 + wn * 128;
            keep_shifted = ncol + 128 > N;   // wave-uniform; N >= 256
            ncol = keep_shifted ? (int64_t)N - 128 : ncol;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                int64_t mrow = m0 + wm * 128 + i * 32 + lrow;
                mrow = mrow < M ? mrow : (int64_t)M - 1;
                const uint8_t* src = rot.mask + mrow * mask_pitch + ncol / 8;
                asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(keep[i]) : "v"(src) : "memory");
            }
        }
        auto block4 = [&](int ks, auto first) {
            constexpr bool FIRST = decltype(first)::value;
            // the four mask-word requests are younger than the stages the first block's steps 0..2 wait for
            constexpr int EX = (FIRST && ROT) ? 4 : 0;
            int lks = ks + 4;
            if (lks == nk) {
                if (t + stride < total_items) {
                    plan_tile(t + stride);
                    lks = 0;
                } else {
                    lks = ks;
                }
            }
            const int lbase = lks + 4 <= nk_real ? lks : nk_real - 4;    // a short last block: the row's final four steps
            const int first_live = ks + 4 > nk_real ? muted : 0;         // this block's steps below it are muted
            const auto sw = [&](int q) { return q < first_live ? 0 : 16; };
            big4_step<0, sizeof(OutT) == 2, FIRST, EX>(plan, smem_bytes, lbase, lbase * 4, sw(0), par, a_off0, a_off1, b_off0, b_off1, a_sc_off, b_sc_off, sh, st, acc);
            big4_step<1, sizeof(OutT) == 2, false, EX>(plan, smem_bytes, lbase + 1, 0, sw(1), par, a_off0, a_off1, b_off0, b_off1, a_sc_off, b_sc_off, sh, st, acc);
            big4_step<2, sizeof(OutT) == 2, false, EX>(plan, smem_bytes, lbase + 2, 0, sw(2), par, a_off0, a_off1, b_off0, b_off1, a_sc_off, b_sc_off, sh, st, acc);
            big4_step<3, sizeof(OutT) == 2>(plan, smem_bytes, lbase + 3, 0, sw(3), par, a_off0, a_off1, b_off0, b_off1, a_sc_off, b_sc_off, sh, st, acc);
            par ^= 1;
        };
        block4(0, std::true_type{});
        for (int ks = 4; ks < nk; ks += 4) block4(ks, std::false_type{});
        stamp();
        if constexpr (sizeof(OutT) == 2) {
            big4_epilogue_bf16<ROT>(acc, alpha, reinterpret_cast<uint16_t*>(c), m0, n0, N, wm, wn, wave, lane, smem_bytes,
                                    rows_valid, cols_valid, rot, keep, keep_shifted);
        } else {
            OutT* dst = splits > 1 ? c + (int64_t)cur_split * M * N : c;
            const float a_eff = splits > 1 ? 1.0f : alpha;
            acc_settle();
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (i * 32 < rows_valid && j * 32 < cols_valid)
                        store_tile<OutT, true>(acc[i][j], a_eff, dst, m0 + wm * 128 + i * 32, n0 + wn * 128 + j * 32 + lrow, N, half);
        }
        stamp();
    }
    // direct-to-LDS loads must not outlive the workgroup's LDS allocation
    __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
}

// c[i] = alpha * (p[0][i] + p[1][i] + ... ) in slab order: the fixed order makes split-K results reproducible
template <typename OutT>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ partial, int splits, int64_t mn,
                                                            float alpha, OutT* __restrict__ c) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    if (i >= mn) return;  // mn is a multiple of 4 (N % 64 == 0)
    float4 acc = *reinterpret_cast<const float4*>(partial + i);
    for (int s = 1; s < splits; ++s) {
        const float4 v = *reinterpret_cast<const float4*>(partial + (int64_t)s * mn + i);
        acc.x += v.x; acc.y += v.y; acc.z += v.z; acc.w += v.w;
    }
    acc.x *= alpha; acc.y *= alpha; acc.z *= alpha; acc.w *= alpha;
    if constexpr (sizeof(OutT) == 4) {
        *reinterpret_cast<float4*>(c + i) = acc;
    } else {
        const uint32_t lo = (uint32_t)f32_to_bf16(acc.x) | ((uint32_t)f32_to_bf16(acc.y) << 16);
        const uint32_t hi = (uint32_t)f32_to_bf16(acc.z) | ((uint32_t)f32_to_bf16(acc.w) << 16);
        *reinterpret_cast<uint2*>(c + i) = make_uint2(lo, hi);
    }
}

// Measurement aid: the block-scaled FP4 matrix instruction alone, on operand bytes taken from `operands`, with no
// memory traffic inside the loop.  What a wave of the GEMM does between its loads: 16 products per iteration on a 4 x 4
// grid of 32 x 32 accumulator blocks.  The rate this reaches on real operand bytes is the chip's ceiling for the
// product at its power limit (the clock it sustains depends on how much the operand bits toggle).
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void mfma_only_kernel(const uint4* __restrict__ operands,
                                                                                                    float* __restrict__ sink, int iters) {
    const int tid = threadIdx.x;
    uint4 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        a[i] = operands[((size_t)blockIdx.x * 8 + i) * 256 + tid];
        b[i] = operands[((size_t)blockIdx.x * 8 + 4 + i) * 256 + tid];
    }
    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;
    const int sc = 0x7f7f7f7f;  // scale 2^0
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const v8i av = v8i{(int)a[i].x, (int)a[i].y, (int)a[i].z, (int)a[i].w, 0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const v8i bv = v8i{(int)b[j].x, (int)b[j].y, (int)b[j].z, (int)b[j].w, 0, 0, 0, 0};
                acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, bv, acc[i][j], 4, 4, 0, sc, 0, sc);
            }
        }
    }
    float sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) sum += acc[i][j][e];
    sink[(size_t)blockIdx.x * 256 + tid] = sum;
}

// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per kernel and device instead of on every launch
constexpr int kMaxDevices = 64;
template <typename Kern>
hipError_t allow_dynamic_lds(Kern kern, int bytes, std::atomic<bool> (&done)[kMaxDevices]) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < kMaxDevices && done[dev].load(std::memory_order_acquire)) return hipSuccess;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && dev >= 0 && dev < kMaxDevices) done[dev].store(true, std::memory_order_release);
    return e;
}

int device_cus() {
    static int cached = 0;  // one GPU model per process
    if (cached > 0) return cached;
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
        n > 0)
        return cached = n;
    return 256;
}

// How many K ranges to cut a GEMM into so that its (tile, range) items fill the CUs: the divisor s of K/512 that
// minimises rounds(s) * steps(s) plus a per-item overhead, each range keeping at least eight K steps.  1 = no split.
int choose_splits(int64_t M, int64_t N, int64_t K, int cus) {
    const int64_t tiles = ((M + kBigM - 1) / kBigM) * ((N + kBigN - 1) / kBigN);
    const int64_t nblk = K / 512;
    if (tiles * 4 >= cus * 3 || nblk < 4) return 1;
    int best = 1;
    double best_cost = 1e30;
    for (int sp = 1; sp <= nblk && sp <= 64; ++sp) {
        if (nblk % sp || (nblk / sp) * 4 < 8) continue;
        const int64_t rounds = (tiles * sp + cus - 1) / cus;
        const double cost = (double)rounds * ((double)(nblk / sp) * 4 + 6.0) + (sp > 1 ? 4.0 + 0.5 * sp : 0.0);
        if (cost < best_cost - 1e-9) {
            best_cost = cost;
            best = sp;
        }
    }
    return best;
}

// late start (units of 1024 cycles) of every other group of workgroups: contractions of at most sixteen K steps per work
// item, where the tile boundary is a third or more of a tile; longer ones neither gain nor lose (within 0.7 %)
int big4_late_start(int64_t K, int splits) { return K / kBK / splits <= 16 ? 6 : 0; }

template <typename OutT, bool ROT = false>
hipError_t launch_big4(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                       const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c, int a_tiled,
                       int b_tiled, int splits, int cus, hipStream_t stream, const RotEpilogue& rot = RotEpilogue{}) {
    auto kern = gemm_mxfp4_tn_big4_kernel<OutT, false, ROT>;
    static std::atomic<bool> lds_allowed[kMaxDevices];
    hipError_t e = allow_dynamic_lds(kern, kBig4SmemBytes, lds_allowed);
    if (e != hipSuccess) return e;
    const int64_t items = ((M + kBigM - 1) / kBigM) * ((N + kBigN - 1) / kBigN) * splits;
    // one workgroup per CU, and a grid that is a multiple of 8 so that item t and t + grid land on the same XCD
    int64_t g = items < cus ? items : cus;
    if (g > 8) g -= g % 8;
    dim3 grid((unsigned)g), block(256);
    kern<<<grid, block, kBig4SmemBytes, stream>>>(a_codes, a_scales, b_codes, b_scales, (int)M, (int)N, (int)K, alpha,
                                                  reinterpret_cast<OutT*>(c), a_tiled, b_tiled, splits, big4_late_start(K, splits), nullptr, rot);
    return hipGetLastError();
}

template <typename OutT>
hipError_t launch_duo(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                      int64_t M, int64_t N, int64_t K, float alpha, void* c, int a_tiled, int b_tiled, int cus, hipStream_t stream) {
    auto kern = gemm_mxfp4_tn_duo_kernel<OutT>;
    static std::atomic<bool> lds_allowed[kMaxDevices];
    hipError_t e = allow_dynamic_lds(kern, kDuoSmemBytes, lds_allowed);
    if (e != hipSuccess) return e;
    const int64_t tiles = ((M + kDuoM - 1) / kDuoM) * ((N + kDuoN - 1) / kDuoN);
    // two workgroups per CU, and a grid that is a multiple of 8 so that tile t and t + grid land on the same XCD
    int64_t g = tiles < 2 * cus ? tiles : 2 * cus;
    if (g > 8) g -= g % 8;
    kern<<<dim3((unsigned)g), dim3(256), kDuoSmemBytes, stream>>>(a_codes, a_scales, b_codes, b_scales, (int)M, (int)N, (int)K, alpha,
                                                                  reinterpret_cast<OutT*>(c), a_tiled, b_tiled);
    return hipGetLastError();
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
            static std::atomic<bool> lds_allowed[kMaxDevices];
            hipError_t e = allow_dynamic_lds(kern, smem, lds_allowed);
            if (e != hipSuccess) return e;
        }
        kern<<<grid, block, smem, stream>>>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, reinterpret_cast<uint16_t*>(c));
    } else {
        auto kern = gemm_mxfp4_tn_kernel<BM, BN, WM, WN, float>;
        if (smem > 48 * 1024) {
            static std::atomic<bool> lds_allowed[kMaxDevices];
            hipError_t e = allow_dynamic_lds(kern, smem, lds_allowed);
            if (e != hipSuccess) return e;
        }
        kern<<<grid, block, smem, stream>>>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, reinterpret_cast<float*>(c));
    }
    return hipGetLastError();
}

}  // namespace

// one launch of the persistent kernel's stamping instantiation (bf16 output, no K ranges); returns its grid size, 0 on
// shapes that kernel does not serve.  stamps: device memory for grid * kPhaseStamps 64-bit values.
int gemm_phase_stamps_per_group() { return kPhaseStamps; }
hipError_t gemm_tile_phases(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes, const uint8_t* b_scales,
                            int64_t M, int64_t N, int64_t K, float alpha, void* c, int a_layout, int b_layout,
                            const uint8_t* rot_mask, unsigned long long* stamps, size_t stamps_bytes, int* grid_out, hipStream_t stream) {
    *grid_out = 0;
    if (!gemm_supports_tiled(M, N, K) || K % 512 || ((reinterpret_cast<uintptr_t>(a_scales) | reinterpret_cast<uintptr_t>(b_scales)) & 15))
        return hipErrorInvalidValue;
    // rot_mask: the instantiation whose epilogue carries the masked inverse rotation (no sign flips, bf16 scale)
    auto kern = rot_mask ? gemm_mxfp4_tn_big4_kernel<uint16_t, true, true> : gemm_mxfp4_tn_big4_kernel<uint16_t, true, false>;
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, kBig4SmemBytes);
    if (e != hipSuccess) return e;
    const int64_t items = ((M + kBigM - 1) / kBigM) * ((N + kBigN - 1) / kBigN);
    const int cus = device_cus();
    int64_t g = items < cus ? items : cus;
    if (g > 8) g -= g % 8;
    if (stamps_bytes < (size_t)g * kPhaseStamps * sizeof(unsigned long long)) return hipErrorInvalidValue;
    kern<<<dim3((unsigned)g), dim3(256), kBig4SmemBytes, stream>>>(a_codes, a_scales, b_codes, b_scales, (int)M, (int)N, (int)K, alpha,
                                                                  reinterpret_cast<uint16_t*>(c), a_layout == LAYOUT_TILED,
                                                                  b_layout == LAYOUT_TILED, 1, big4_late_start(K, 1), stamps,
                                                                  RotEpilogue{rot_mask, 0u, hadamard_scale(32, BF16)});
    *grid_out = (int)g;
    return hipGetLastError();
}

// one workgroup (four waves, one per SIMD) per CU; reads blocks * 32 KiB of operands, writes blocks * 256 floats
int mfma_only_blocks() { return device_cus(); }
hipError_t mfma_only(const uint8_t* operands, float* sink, int iters, hipStream_t stream) {
    mfma_only_kernel<<<dim3((unsigned)device_cus()), dim3(256), 0, stream>>>(reinterpret_cast<const uint4*>(operands), sink, iters);
    return hipGetLastError();
}

// Shapes the 256x256-tile kernels serve (they also read tiled operands): extents multiples of 64 and at least one
// full tile wide, K a multiple of 128; tiles hanging over the edge of M or N compute on clamped rows and store nothing there.
bool gemm_supports_tiled(int64_t M, int64_t N, int64_t K) {
    return M % 64 == 0 && N % 64 == 0 && M >= kBigM && N >= kBigN && K > 0 && K % kBK == 0 && M < (1 << 30) && N < (1 << 30) &&
           K < (1 << 30);
}

// bytes of scratch with which gemm_mxfp4_tn cuts this shape into K ranges (0: it would not)
size_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (!gemm_supports_tiled(M, N, K) || K % 512 || K <= kDuoMaxK) return 0;
    const int sp = choose_splits(M, N, K, device_cus());
    return sp > 1 ? (size_t)sp * (size_t)M * (size_t)N * sizeof(float) : 0;
}

hipError_t gemm_mxfp4_tn(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                         const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype,
                         int a_layout, int b_layout, void* workspace, size_t workspace_bytes, hipStream_t stream) {
    return gemm_mxfp4_tn_rotated(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, c_dtype, a_layout, b_layout, workspace,
                                 workspace_bytes, nullptr, 0u, F32, c_dtype, nullptr, stream);
}

// whether gemm_mxfp4_tn_rotated would apply the rotation itself for these arguments: in the epilogue of an uncut product
// (bf16 in and out), or in the reduction of a product it cuts into K ranges
bool gemm_will_rotate(const uint8_t* a_scales, const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, int c_dtype, int rot_out_dtype,
                      const void* workspace, size_t workspace_bytes) {
    if (!gemm_supports_tiled(M, N, K) || K <= kDuoMaxK) return false;
    if (rot_out_dtype != c_dtype && !(c_dtype == BF16 && rot_out_dtype == F32)) return false;
    const int64_t nk_real = K / kBK, nk_pad = (nk_real + 3) & ~(int64_t)3;
    const bool persistent_ok = K % 512 == 0 ? ((reinterpret_cast<uintptr_t>(a_scales) | reinterpret_cast<uintptr_t>(b_scales)) & 15) == 0
                                            : (nk_real >= 4 && (nk_pad - nk_real) * 3 <= nk_real);
    if (!persistent_ok) return false;
    int sp = workspace && K % 512 == 0 ? choose_splits(M, N, K, device_cus()) : 1;
    if (sp > 1 && ((size_t)sp * M * N * sizeof(float) > workspace_bytes || (reinterpret_cast<uintptr_t>(workspace) & 15))) sp = 1;
    return sp > 1 || (c_dtype == BF16 && rot_out_dtype == BF16);
}

// The product, with the layer's masked inverse Hadamard rotation (blocks of 32 along N) applied to the result before it is
// stored when `rot_mask` is given and gemm_will_rotate() holds: in the persistent kernel's bf16 epilogue, or in the ordered
// reduction of the K ranges.  *rotated tells which (true: c holds the rotated result in rot_out_dtype; false: c holds the
// plain product in c_dtype and the caller runs the rotation as a kernel of its own).
hipError_t gemm_mxfp4_tn_rotated(const uint8_t* a_codes, const uint8_t* a_scales, const uint8_t* b_codes,
                                 const uint8_t* b_scales, int64_t M, int64_t N, int64_t K, float alpha, void* c, int c_dtype,
                                 int a_layout, int b_layout, void* workspace, size_t workspace_bytes, const uint8_t* rot_mask,
                                 uint32_t rot_signs, int rot_scale_dtype, int rot_out_dtype, bool* rotated, hipStream_t stream) {
    if (rotated) *rotated = false;
    if (M == 0 || N == 0) return hipSuccess;
    const int at = a_layout == LAYOUT_TILED, bt = b_layout == LAYOUT_TILED;
    const bool big_ok = gemm_supports_tiled(M, N, K);
    if ((at || bt) && !big_ok) return hipErrorInvalidValue;
    // The persistent kernel walks K in blocks of four steps: K % 512 == 0 directly (scale rows are then 16-byte aligned
    // like their base), other multiples of 128 with up to three muted steps in the last block when those are at most a
    // third of the real ones (K = 1152 and 1664 gain 3-5 % over a kernel without muted steps); their 16-byte scale
    // requests start at 4-byte aligned addresses.  Every multiple of 128 above 768 qualifies; up to 768 the contraction is
    // so short that the tile boundary dominates and the two-workgroups-per-CU kernel is faster (measured at 32768 tokens:
    // 640 x 640 15 against 23 us, 3456 x 640 70 against 82 us; at K = 1536 it is 13-25 % slower than the persistent kernel).
    const int64_t nk_real = K / kBK, nk_pad = (nk_real + 3) & ~(int64_t)3;
    const bool persistent_ok = K % 512 == 0 ? ((reinterpret_cast<uintptr_t>(a_scales) | reinterpret_cast<uintptr_t>(b_scales)) & 15) == 0
                                            : (nk_real >= 4 && (nk_pad - nk_real) * 3 <= nk_real);
    // K % 128 == 64 (the 30 M Llama's hidden width 1728): the two-workgroup kernel closes such a contraction with a half
    // step.  Row-major operands (the tiled layout does not exist for these K); a c that is only 4-byte aligned, which the
    // interface accepts at these shapes, stays on the generic kernel.
    const bool half_ok = !at && !bt && K % kBK == 64 && K >= 192 && gemm_supports_tiled(M, N, K - 64) &&
                         (reinterpret_cast<uintptr_t>(c) & 15) == 0;
    if (half_ok) {
        const int cus = device_cus();
        if (c_dtype == BF16) return launch_duo<uint16_t>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, 0, 0, cus, stream);
        return launch_duo<float>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, 0, 0, cus, stream);
    }
    if (big_ok && (K <= kDuoMaxK || !persistent_ok)) {
        // short contraction: two 256 x 128 workgroups per CU hide each other's tile boundaries (also the fallback for scale
        // arrays that are not 16-byte aligned, which the persistent kernel's 16-byte scale requests need when K % 512 == 0)
        const int cus = device_cus();
        if (c_dtype == BF16) return launch_duo<uint16_t>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, at, bt, cus, stream);
        return launch_duo<float>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, at, bt, cus, stream);
    }
    if (big_ok && persistent_ok) {
        const int cus = device_cus();
        int sp = workspace && K % 512 == 0 ? choose_splits(M, N, K, cus) : 1;  // K ranges are whole blocks of four steps
        if (sp > 1 && ((size_t)sp * M * N * sizeof(float) > workspace_bytes || (reinterpret_cast<uintptr_t>(workspace) & 15))) sp = 1;
        if (sp > 1) {
            // partial sums per K range in fp32 (plain accumulator layout), then one ordered reduction
            hipError_t e = launch_big4<float>(a_codes, a_scales, b_codes, b_scales, M, N, K, 1.0f, workspace, at, bt, sp, cus, stream);
            if (e != hipSuccess) return e;
            const int64_t mn = M * N;
            if (rot_mask && rotated && (rot_out_dtype == c_dtype || (c_dtype == BF16 && rot_out_dtype == F32))) {
                *rotated = true;
                return splitk_reduce_rotated(static_cast<const float*>(workspace), sp, mn, alpha, c_dtype, rot_mask, rot_signs, rot_scale_dtype,
                                             c, rot_out_dtype, stream);
            }
            dim3 grid((unsigned)((mn / 4 + 255) / 256)), block(256);
            if (c_dtype == BF16)
                splitk_reduce_kernel<uint16_t><<<grid, block, 0, stream>>>(static_cast<const float*>(workspace), sp, mn, alpha, static_cast<uint16_t*>(c));
            else
                splitk_reduce_kernel<float><<<grid, block, 0, stream>>>(static_cast<const float*>(workspace), sp, mn, alpha, static_cast<float*>(c));
            return hipGetLastError();
        }
        if (c_dtype == BF16 && rot_out_dtype == BF16 && rot_mask && rotated) {
            *rotated = true;
            const RotEpilogue rot{rot_mask, rot_signs, hadamard_scale(32, rot_scale_dtype)};
            return launch_big4<uint16_t, true>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, at, bt, 1, cus, stream, rot);
        }
        if (c_dtype == BF16) return launch_big4<uint16_t>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, at, bt, 1, cus, stream);
        return launch_big4<float>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, at, bt, 1, cus, stream);
    }
    return launch_gemm<128, 128, 64, 64>(a_codes, a_scales, b_codes, b_scales, M, N, K, alpha, c, c_dtype, stream);
}

}  // namespace qm
