// Backward passes of the producers that are fused into the forward quantizer: RMSNorm
// (src/models/llama.py:64-75 of the reference) and the SwiGLU product (llama.py:113-114).  Floating-point kernels:
// they follow the formulas autograd derives for those lines, not a bit-exact instruction order.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qm_kernels.h"
#include "qm_math.h"

namespace qm {

namespace {

typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

template <typename T>
__device__ __forceinline__ float4 load4(const T* p) {
    if constexpr (sizeof(T) == 2) {
        const uint2 raw = *reinterpret_cast<const uint2*>(p);
        return make_float4(u2f(raw.x << 16), u2f(raw.x & 0xffff0000u), u2f(raw.y << 16), u2f(raw.y & 0xffff0000u));
    } else {
        return *reinterpret_cast<const float4*>(p);
    }
}
template <typename T>
__device__ __forceinline__ void store4(T* p, float4 v) {
    if constexpr (sizeof(T) == 2) {
        const uint32_t lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v.x, v.y}, v2bf));
        const uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v.z, v.w}, v2bf));
        *reinterpret_cast<uint2*>(p) = make_uint2(lo, hi);
    } else {
        *reinterpret_cast<float4*>(p) = v;
    }
}

// The straight-through backward of the forward quantizer (masked inverse rotation, Hadamard block 32,
// src/models/quantization/quantizers/mxfp4.py:143-146) on four consecutive elements of a lane; the eight lanes that hold
// a group of 32 cooperate.  The same operations on the same pairs as the stand-alone kernel (mask factor, column sign,
// ascending butterfly strides, one multiply by c, rounding to the gradient's dtype), hence the same bits.
struct InverseRotation {
    const uint8_t* maskbits;  // null: the gradient arrives already rotated back
    uint32_t sign_word;
    float c;
};
__device__ __forceinline__ float quad_xor1(float v) { return u2f((uint32_t)__builtin_amdgcn_mov_dpp((int)f2u(v), 0xB1, 0xF, 0xF, true)); }
__device__ __forceinline__ float quad_xor2(float v) { return u2f((uint32_t)__builtin_amdgcn_mov_dpp((int)f2u(v), 0x4E, 0xF, 0xF, true)); }
// keep: bit i = clip-mask bit of element elem + i (the caller has fetched the mask byte)
template <bool ROUND_BF16>
__device__ __forceinline__ float4 inverse_rotate_quad_bits(float4 g, const InverseRotation& rot, int64_t elem, uint32_t keep) {
    const int q = (int)(elem >> 2) & 7;                                            // the lane's place in its group
    const uint32_t sign = rot.sign_word >> (q * 4);
    float v[4] = {g.x, g.y, g.z, g.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float x = v[i] * (((keep >> i) & 1u) ? 1.0f : 0.0f);
        v[i] = u2f(f2u(x) ^ (((sign >> i) & 1u) << 31));
    }
#pragma unroll
    for (int h = 1; h < 4; h <<= 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            if (i & h) continue;
            const float a = v[i], b = v[i + h];
            v[i] = a + b;
            v[i + h] = a - b;
        }
    }
#pragma unroll
    for (int m = 1; m < 8; m <<= 1) {  // lower lane of a butterfly: own + partner; upper lane: partner - own
        const uint32_t flip = (q & m) ? 0x80000000u : 0u;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float p = m == 1 ? quad_xor1(v[i]) : (m == 2 ? quad_xor2(v[i]) : __shfl_xor(v[i], 4, 64));
            v[i] = p + u2f(f2u(v[i]) ^ flip);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = v[i] * rot.c;
    if constexpr (ROUND_BF16) {
#pragma unroll
        for (int i = 0; i < 4; i += 2) {
            const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[i], v[i + 1]}, v2bf));
            v[i] = u2f(w << 16);
            v[i + 1] = u2f(w & 0xffff0000u);
        }
    }
    return make_float4(v[0], v[1], v[2], v[3]);
}

template <bool ROUND_BF16>
__device__ __forceinline__ float4 inverse_rotate_quad(float4 g, const InverseRotation& rot, int64_t elem) {
    return inverse_rotate_quad_bits<ROUND_BF16>(g, rot, elem, (uint32_t)rot.maskbits[elem >> 3] >> (elem & 4));
}

// rows one workgroup walks: at most 1024 workgroups (one resident round on the chip), so at most 1024 partial rows
inline int rows_per_block(int64_t rows) { return (int)((rows + 1023) / 1024 > 0 ? (rows + 1023) / 1024 : 1); }

// y = x f g with f = (mean(x^2) + eps)^-1/2:
//   dx_i = f g_i gy_i - x_i f^3 / cols * sum_j gy_j g_j x_j,      dgain_i = sum_rows gy_i x_i f.
// A workgroup walks rpb rows, RB at a time; thread t owns columns 4 (t + 256 k) .. +3 of each, keeps the rows in registers
// between the reduction and the update, and adds its columns' gain-gradient terms over the rows: one partial row per workgroup.
template <typename TG, typename TX, int NK, int RB>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(const TG* __restrict__ gy, const TX* __restrict__ x,
                                                          const float* __restrict__ gain, const float* __restrict__ factor,
                                                          int64_t rows, int cols, int rpb, InverseRotation rot,
                                                          const TX* __restrict__ skip, TX* __restrict__ dx,
                                                          uint16_t* __restrict__ dx_bf16, float* __restrict__ partial) {
    __shared__ float wave_sums[2][RB][4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t r0 = (int64_t)blockIdx.x * rpb;
    const int64_t r1 = r0 + rpb < rows ? r0 + rpb : rows;
    float4 acc[NK], w[NK];
#pragma unroll
    for (int k = 0; k < NK; ++k) {
        const int col = (k * 256 + (int)threadIdx.x) * 4;
        acc[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        w[k] = col < cols ? *reinterpret_cast<const float4*>(gain + col) : acc[k];
    }
    int parity = 0;
    for (int64_t rb = r0; rb < r1; rb += RB, parity ^= 1) {  // RB rows in flight at a time
        float f[RB], s[RB];
        float4 gk[RB][NK], xk[RB][NK];
#pragma unroll
        for (int j = 0; j < RB; ++j) {
            const int64_t r = rb + j < r1 ? rb + j : r1 - 1;  // a repeated last row is computed and not stored
            f[j] = factor[r];
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int col = (k * 256 + (int)threadIdx.x) * 4;
                if (col < cols) {  // cols % 32 == 0: the eight lanes of a group of 32 are in or out together
                    gk[j][k] = load4(gy + r * cols + col);
                    if (rot.maskbits) gk[j][k] = inverse_rotate_quad<sizeof(TG) == 2>(gk[j][k], rot, r * cols + col);
                    xk[j][k] = load4(x + r * cols + col);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < RB; ++j) {
            s[j] = 0.0f;
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int col = (k * 256 + (int)threadIdx.x) * 4;
                if (col < cols) {
                    const float4 g = gk[j][k], v = xk[j][k];
                    s[j] += g.x * w[k].x * v.x + g.y * w[k].y * v.y + g.z * w[k].z * v.z + g.w * w[k].w * v.w;
                    if (rb + j < r1) {
                        acc[k].x += g.x * v.x * f[j]; acc[k].y += g.y * v.y * f[j];
                        acc[k].z += g.z * v.z * f[j]; acc[k].w += g.w * v.w * f[j];
                    }
                }
            }
#pragma unroll
            for (int m = 32; m >= 1; m >>= 1) s[j] += __shfl_xor(s[j], m, 64);
            // two sets of slots: a wave may start the next rows while another still reads these
            if (lane == 0) wave_sums[parity][j][wave] = s[j];
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < RB; ++j) {
            if (rb + j >= r1) break;
            const float* slot = wave_sums[parity][j];
            const float coef = f[j] * f[j] * f[j] * ((slot[0] + slot[1]) + (slot[2] + slot[3])) / (float)cols;
#pragma unroll
            for (int k = 0; k < NK; ++k) {
                const int col = (k * 256 + (int)threadIdx.x) * 4;
                if (col < cols) {
                    const float4 g = gk[j][k], v = xk[j][k];
                    const float fj = f[j];
                    float4 d = make_float4(fj * g.x * w[k].x - v.x * coef, fj * g.y * w[k].y - v.y * coef,
                                           fj * g.z * w[k].z - v.z * coef, fj * g.w * w[k].w - v.w * coef);
                    if (skip) {  // the gradient that reaches x past the norm (the residual connection), added as autograd would
                        if constexpr (sizeof(TX) == 2) {  // a bf16 gradient is rounded before the sum, as a stored tensor is
                            const uint32_t lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{d.x, d.y}, v2bf));
                            const uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{d.z, d.w}, v2bf));
                            d = make_float4(u2f(lo << 16), u2f(lo & 0xffff0000u), u2f(hi << 16), u2f(hi & 0xffff0000u));
                        }
                        const float4 sk = load4(skip + (rb + j) * cols + col);
                        d = make_float4(d.x + sk.x, d.y + sk.y, d.z + sk.z, d.w + sk.w);
                    }
                    store4(dx + (rb + j) * cols + col, d);
                    if (dx_bf16) store4(dx_bf16 + (rb + j) * cols + col, d);  // the gradient of a bf16 summand of x
                }
            }
        }
    }
#pragma unroll
    for (int k = 0; k < NK; ++k) {
        const int col = (k * 256 + (int)threadIdx.x) * 4;
        if (col < cols) *reinterpret_cast<float4*>(partial + (int64_t)blockIdx.x * cols + col) = acc[k];
    }
}

// The same computation for rows of at most 256 NK columns, one wave per row and no barrier in the row loop: a wave
// requests its next row (gradient, mask bytes, x, residual gradient) before it works on the current one, so every wave
// has a row in flight all the time, and the row's mask bits arrive as one dword per lane and reach their lanes by a
// shuffle instead of one byte load per quad (at 1536 columns, with residual gradient and bf16 copy: 5.1 TB/s against the
// 3.8 of the cooperative kernel above, which alternates between requesting and computing).
// Lane l owns columns 4 (l + 64 k) .. +3; the four waves of a workgroup add their gain-gradient terms in wave order
// at the end: one partial row per workgroup.
constexpr int kRowWaveGrid = 512;  // workgroups: two waves per SIMD on 256 CUs

template <typename TG, typename TX, int NK>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void rmsnorm_bwd_rows_kernel(const TG* __restrict__ gy, const TX* __restrict__ x,
                                                               const float* __restrict__ gain,
                                                               const float* __restrict__ factor, int64_t rows, int cols,
                                                               InverseRotation rot, const TX* __restrict__ skip,
                                                               TX* __restrict__ dx, uint16_t* __restrict__ dx_bf16,
                                                               float* __restrict__ partial) {
    __shared__ float4 wave_acc[3][NK][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int64_t stride = (int64_t)gridDim.x * 4;
    struct Row {
        float4 g[NK], x[NK], s[NK];
        uint32_t maskword;  // lane l: clip-mask bits of the row's columns 32 l .. 32 l + 31
        float f;
    };
    float4 acc[NK], w[NK];
#pragma unroll
    for (int k = 0; k < NK; ++k) {
        const int col = (k * 64 + lane) * 4;
        acc[k] = make_float4(0.f, 0.f, 0.f, 0.f);
        w[k] = col < cols ? *reinterpret_cast<const float4*>(gain + col) : acc[k];
    }
    const auto request = [&](int64_t r, Row& row) {
        row.f = factor[r];
        // the row's mask bits in one dword per lane (rows start on 4-byte boundaries: cols % 32 == 0)
        row.maskword = 0u;
        if (rot.maskbits && lane * 32 < cols) row.maskword = reinterpret_cast<const uint32_t*>(rot.maskbits + r * (cols / 8))[lane];
#pragma unroll
        for (int k = 0; k < NK; ++k) {
            const int col = (k * 64 + lane) * 4;
            if (col < cols) {  // cols % 32 == 0: the eight lanes of a group of 32 are in or out together
                const int64_t e = r * cols + col;
                row.g[k] = load4(gy + e);
                row.x[k] = load4(x + e);
                if (skip) row.s[k] = load4(skip + e);
            }
        }
    };
    const auto work = [&](int64_t r, Row& row) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < NK; ++k) {
            const int col = (k * 64 + lane) * 4;
            // the group's mask dword sits in lane 8 k + lane / 8; the lane's four bits are nibble lane % 8 of it
            const uint32_t word = rot.maskbits ? (uint32_t)__shfl((int)row.maskword, 8 * k + (lane >> 3), 64) : 0u;
            if (col < cols) {
                if (rot.maskbits) row.g[k] = inverse_rotate_quad_bits<sizeof(TG) == 2>(row.g[k], rot, r * cols + col, word >> (4 * (lane & 7)));
                const float4 g = row.g[k], v = row.x[k];
                s += g.x * w[k].x * v.x + g.y * w[k].y * v.y + g.z * w[k].z * v.z + g.w * w[k].w * v.w;
                acc[k].x += g.x * v.x * row.f; acc[k].y += g.y * v.y * row.f;
                acc[k].z += g.z * v.z * row.f; acc[k].w += g.w * v.w * row.f;
            }
        }
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1) s += __shfl_xor(s, m, 64);
        const float fj = row.f;
        const float coef = fj * fj * fj * s / (float)cols;
#pragma unroll
        for (int k = 0; k < NK; ++k) {
            const int col = (k * 64 + lane) * 4;
            if (col < cols) {
                const float4 g = row.g[k], v = row.x[k];
                float4 d = make_float4(fj * g.x * w[k].x - v.x * coef, fj * g.y * w[k].y - v.y * coef,
                                       fj * g.z * w[k].z - v.z * coef, fj * g.w * w[k].w - v.w * coef);
                if (skip) {  // as in the cooperative kernel: a bf16 gradient is rounded before the sum
                    if constexpr (sizeof(TX) == 2) {
                        const uint32_t lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{d.x, d.y}, v2bf));
                        const uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{d.z, d.w}, v2bf));
                        d = make_float4(u2f(lo << 16), u2f(lo & 0xffff0000u), u2f(hi << 16), u2f(hi & 0xffff0000u));
                    }
                    const float4 sk = row.s[k];
                    d = make_float4(d.x + sk.x, d.y + sk.y, d.z + sk.z, d.w + sk.w);
                }
                store4(dx + r * cols + col, d);
                if (dx_bf16) store4(dx_bf16 + r * cols + col, d);
            }
        }
    };
    Row a, b;
    int64_t r = (int64_t)blockIdx.x * 4 + wave;
    if (r < rows) request(r, a);
    while (r < rows) {  // two rows per trip so that the buffers swap roles without register copies
        if (r + stride < rows) request(r + stride, b);
        work(r, a);
        r += stride;
        if (r >= rows) break;
        if (r + stride < rows) request(r + stride, a);
        work(r, b);
        r += stride;
    }
    // gain-gradient terms of the workgroup's rows: wave 0's plus waves 1, 2, 3's in that order
    if (wave > 0) {
#pragma unroll
        for (int k = 0; k < NK; ++k) wave_acc[wave - 1][k][lane] = acc[k];
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
        for (int k = 0; k < NK; ++k) {
            const int col = (k * 64 + lane) * 4;
            float4 t = acc[k];
#pragma unroll
            for (int o = 0; o < 3; ++o) {
                const float4 u = wave_acc[o][k][lane];
                t = make_float4(t.x + u.x, t.y + u.y, t.z + u.z, t.w + u.w);
            }
            if (col < cols) *reinterpret_cast<float4*>(partial + (int64_t)blockIdx.x * cols + col) = t;
        }
    }
}

// dgain[c] = sum over the n partial rows, in a fixed order: 16 waves take rows w, w+16, ...; their sums are added in
// wave order.  One workgroup of 1024 threads per 64 columns.
__global__ __launch_bounds__(1024) void column_sum_kernel(const float* __restrict__ partial, int n, int cols,
                                                          float* __restrict__ out) {
    __shared__ float sums[16][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int col = blockIdx.x * 64 + lane;
    float s = 0.0f;
    if (col < cols) {
#pragma unroll 8
        for (int r = wave; r < n; r += 16) s += partial[(int64_t)r * cols + col];
    }
    sums[wave][lane] = s;
    __syncthreads();
    if (wave == 0 && col < cols) {
        float t = sums[0][lane];
#pragma unroll
        for (int w = 1; w < 16; ++w) t += sums[w][lane];
        out[col] = t;
    }
}

// h = silu(up) * gate:  d_gate = g silu(up),  d_up = g gate s (1 + up (1 - s)),  s = 1 / (1 + e^-up).
// A tensor of bf16 rounds where autograd's bf16 ops would: silu(up), g * gate, and the two results.
template <typename TG, typename TH>
__global__ __launch_bounds__(256) void swiglu_bwd_kernel(const TG* __restrict__ g, const TH* __restrict__ h12,
                                                         int64_t rows, int64_t hidden, InverseRotation rot,
                                                         TH* __restrict__ d_h12) {
    const int64_t quads_per_row = hidden / 4;
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= rows * quads_per_row) return;
    const int64_t row = q / quads_per_row, col = (q - row * quads_per_row) * 4;
    float4 gv = load4(g + row * hidden + col);
    if (rot.maskbits) gv = inverse_rotate_quad<sizeof(TG) == 2>(gv, rot, row * hidden + col);  // hidden % 32 == 0 then
    const float4 up = load4(h12 + row * 2 * hidden + col), gate = load4(h12 + row * 2 * hidden + hidden + col);
    const float G[4] = {gv.x, gv.y, gv.z, gv.w}, U[4] = {up.x, up.y, up.z, up.w}, A[4] = {gate.x, gate.y, gate.z, gate.w};
    float du[4], da[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-U[i] * 1.44269504f));
        float a = U[i] * s, t = G[i] * A[i];
        if constexpr (sizeof(TH) == 2) {
            a = bf16_to_f32(f32_to_bf16(a));
            t = bf16_to_f32(f32_to_bf16(t));
        }
        da[i] = G[i] * a;
        du[i] = t * s * (1.0f + U[i] * (1.0f - s));
    }
    store4(d_h12 + row * 2 * hidden + col, make_float4(du[0], du[1], du[2], du[3]));
    store4(d_h12 + row * 2 * hidden + hidden + col, make_float4(da[0], da[1], da[2], da[3]));
}

// Eight consecutive elements per lane: 16-byte accesses for bf16 tensors, and the clip mask of the lane's elements is
// exactly one byte.  The four lanes that hold a group of 32 cooperate as in the stand-alone inverse rotation (three
// butterfly strides inside the lane, two across lanes): the same operations on the same pairs, hence the same bits.
template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        const uint4 raw = *reinterpret_cast<const uint4*>(p);
        const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            v[2 * i] = u2f(w[i] << 16);
            v[2 * i + 1] = u2f(w[i] & 0xffff0000u);
        }
    } else {
        const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
        v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
}
template <typename T>
__device__ __forceinline__ void store8(T* p, const float (&v)[8]) {
    if constexpr (sizeof(T) == 2) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[2 * i], v[2 * i + 1]}, v2bf));
        *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
    } else {
        *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
        *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
    }
}
template <bool ROUND_BF16>
__device__ __forceinline__ void inverse_rotate_oct(float (&v)[8], const InverseRotation& rot, int64_t elem) {
    const int lic = (int)(elem >> 3) & 3;  // the lane's place in its group
    const uint32_t keep = (uint32_t)rot.maskbits[elem >> 3];
    const uint32_t sign = rot.sign_word >> (lic * 8);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float x = v[i] * (((keep >> i) & 1u) ? 1.0f : 0.0f);
        v[i] = u2f(f2u(x) ^ (((sign >> i) & 1u) << 31));
    }
#pragma unroll
    for (int h = 1; h < 8; h <<= 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (i & h) continue;
            const float a = v[i], b = v[i + h];
            v[i] = a + b;
            v[i + h] = a - b;
        }
    }
#pragma unroll
    for (int m = 1; m < 4; m <<= 1) {  // lower lane of a butterfly: own + partner; upper lane: partner - own
        const uint32_t flip = (lic & m) ? 0x80000000u : 0u;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float p = m == 1 ? quad_xor1(v[i]) : quad_xor2(v[i]);
            v[i] = p + u2f(f2u(v[i]) ^ flip);
        }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = v[i] * rot.c;
    if constexpr (ROUND_BF16) {
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
            const uint32_t w = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2f{v[i], v[i + 1]}, v2bf));
            v[i] = u2f(w << 16);
            v[i + 1] = u2f(w & 0xffff0000u);
        }
    }
}

// hidden % 8 == 0: the same arithmetic per element as swiglu_bwd_kernel, half as many memory instructions per element
// (used when the gradient arrives rotated: there the mask byte per quad of the other kernel is what it saves)
template <typename TG, typename TH>
__global__ __launch_bounds__(256) void swiglu_bwd_oct_kernel(const TG* __restrict__ g, const TH* __restrict__ h12,
                                                             int64_t rows, int64_t hidden, InverseRotation rot,
                                                             TH* __restrict__ d_h12) {
    const int64_t octs_per_row = hidden / 8;
    const int64_t q = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= rows * octs_per_row) return;
    const int64_t row = q / octs_per_row, col = (q - row * octs_per_row) * 8;
    float G[8], U[8], A[8], du[8], da[8];
    load8(g + row * hidden + col, G);
    load8(h12 + row * 2 * hidden + col, U);
    load8(h12 + row * 2 * hidden + hidden + col, A);
    if (rot.maskbits) inverse_rotate_oct<sizeof(TG) == 2>(G, rot, row * hidden + col);  // hidden % 32 == 0 then
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float s = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-U[i] * 1.44269504f));
        float a = U[i] * s, t = G[i] * A[i];
        if constexpr (sizeof(TH) == 2) {
            a = bf16_to_f32(f32_to_bf16(a));
            t = bf16_to_f32(f32_to_bf16(t));
        }
        da[i] = G[i] * a;
        du[i] = t * s * (1.0f + U[i] * (1.0f - s));
    }
    store8(d_h12 + row * 2 * hidden + col, du);
    store8(d_h12 + row * 2 * hidden + hidden + col, da);
}

// one wave per row for rows of at most 1536 columns (see rmsnorm_bwd_rows_kernel), the cooperative kernel above that
inline bool rows_kernel_serves(int64_t cols) { return cols <= 1536; }
int64_t rmsnorm_bwd_blocks(int64_t rows, int64_t cols) {
    if (rows_kernel_serves(cols)) return (rows + 3) / 4 < kRowWaveGrid ? (rows + 3) / 4 : kRowWaveGrid;
    return (rows + rows_per_block(rows) - 1) / rows_per_block(rows);
}

template <typename TG, typename TX>
void launch_rmsnorm_bwd(const void* gy, const void* x, const float* gain, const float* factor, int64_t rows, int cols,
                        const InverseRotation& rot, const void* skip, void* dx, void* dx_bf16, float* partial,
                        hipStream_t stream) {
    const dim3 grid((unsigned)rmsnorm_bwd_blocks(rows, cols)), block(256);
    const int rpb = rows_per_block(rows);
    const TG* g = reinterpret_cast<const TG*>(gy);
    const TX* xp = reinterpret_cast<const TX*>(x);
    TX* dxp = reinterpret_cast<TX*>(dx);
    const TX* sk = reinterpret_cast<const TX*>(skip);
    uint16_t* dxb = reinterpret_cast<uint16_t*>(dx_bf16);
    if (cols <= 768) rmsnorm_bwd_rows_kernel<TG, TX, 3><<<grid, block, 0, stream>>>(g, xp, gain, factor, rows, cols, rot, sk, dxp, dxb, partial);
    else if (rows_kernel_serves(cols)) rmsnorm_bwd_rows_kernel<TG, TX, 6><<<grid, block, 0, stream>>>(g, xp, gain, factor, rows, cols, rot, sk, dxp, dxb, partial);
    else if (cols <= 2048) rmsnorm_bwd_kernel<TG, TX, 2, 4><<<grid, block, 0, stream>>>(g, xp, gain, factor, rows, cols, rpb, rot, sk, dxp, reinterpret_cast<uint16_t*>(dx_bf16), partial);
    else if (cols <= 4096) rmsnorm_bwd_kernel<TG, TX, 4, 2><<<grid, block, 0, stream>>>(g, xp, gain, factor, rows, cols, rpb, rot, sk, dxp, reinterpret_cast<uint16_t*>(dx_bf16), partial);
    else rmsnorm_bwd_kernel<TG, TX, 8, 1><<<grid, block, 0, stream>>>(g, xp, gain, factor, rows, cols, rpb, rot, sk, dxp, reinterpret_cast<uint16_t*>(dx_bf16), partial);
}

}  // namespace

size_t rmsnorm_backward_workspace_bytes(int64_t rows, int64_t cols) {
    return (size_t)rmsnorm_bwd_blocks(rows, cols) * (size_t)cols * sizeof(float);
}

// cols <= 8192, cols % 32 == 0; workspace: rmsnorm_backward_workspace_bytes(rows, cols) bytes, 16-byte aligned.
// maskbits != null: gy is the gradient w.r.t. the quantizer's rotated output and is rotated back on the fly.
// skip != null: [rows, cols] of x's dtype, added to dx (the gradient of a residual connection around the norm).
// dx_bf16 != null: a second copy of dx rounded to bf16 (the gradient of a bf16 tensor that was added into x).
hipError_t rmsnorm_backward(const void* gy, int gy_dtype, const void* x, int x_dtype, const float* gain,
                            const float* factor, int64_t rows, int64_t cols, const uint8_t* maskbits, uint32_t sign_word,
                            int scale_dtype, const void* skip, void* dx, void* dx_bf16, float* dgain, void* workspace,
                            hipStream_t stream) {
    if (cols == 0) return hipSuccess;
    float* partial = reinterpret_cast<float*>(workspace);
    const InverseRotation rot{maskbits, sign_word, hadamard_scale(32, scale_dtype)};
    if (rows == 0) {}  // no rows: the column sums below write zeros
    else if (gy_dtype == BF16 && x_dtype == BF16) launch_rmsnorm_bwd<uint16_t, uint16_t>(gy, x, gain, factor, rows, (int)cols, rot, skip, dx, dx_bf16, partial, stream);
    else if (gy_dtype == BF16) launch_rmsnorm_bwd<uint16_t, float>(gy, x, gain, factor, rows, (int)cols, rot, skip, dx, dx_bf16, partial, stream);
    else if (x_dtype == BF16) launch_rmsnorm_bwd<float, uint16_t>(gy, x, gain, factor, rows, (int)cols, rot, skip, dx, dx_bf16, partial, stream);
    else launch_rmsnorm_bwd<float, float>(gy, x, gain, factor, rows, (int)cols, rot, skip, dx, dx_bf16, partial, stream);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    column_sum_kernel<<<dim3((unsigned)((cols + 63) / 64)), dim3(1024), 0, stream>>>(partial, (int)rmsnorm_bwd_blocks(rows, cols),
                                                                                    (int)cols, dgain);
    return hipGetLastError();
}

// hidden % 4 == 0 (% 32 with maskbits); maskbits as for rmsnorm_backward
hipError_t swiglu_backward(const void* g, int g_dtype, const void* h12, int dtype, int64_t rows, int64_t hidden,
                           const uint8_t* maskbits, uint32_t sign_word, int scale_dtype, void* d_h12, hipStream_t stream) {
    if (rows == 0 || hidden == 0) return hipSuccess;
    const InverseRotation rot{maskbits, sign_word, hadamard_scale(32, scale_dtype)};
    // with the inverse rotation the octet kernel is 10 % faster (232 against 259 us at 32768 x 4096), without it 4 % slower
    const bool oct = maskbits && hidden % 8 == 0;
    const dim3 grid((unsigned)((rows * (hidden / (oct ? 8 : 4)) + 255) / 256)), block(256);
    const auto go = [&](auto tg, auto th) {
        using TG = decltype(tg);
        using TH = decltype(th);
        const TG* gp = reinterpret_cast<const TG*>(g);
        const TH* hp = reinterpret_cast<const TH*>(h12);
        TH* dp = reinterpret_cast<TH*>(d_h12);
        if (oct) swiglu_bwd_oct_kernel<TG, TH><<<grid, block, 0, stream>>>(gp, hp, rows, hidden, rot, dp);
        else swiglu_bwd_kernel<TG, TH><<<grid, block, 0, stream>>>(gp, hp, rows, hidden, rot, dp);
    };
    if (g_dtype == BF16 && dtype == BF16) go(uint16_t{}, uint16_t{});
    else if (g_dtype == BF16) go(uint16_t{}, float{});
    else if (dtype == BF16) go(float{}, uint16_t{});
    else go(float{}, float{});
    return hipGetLastError();
}

}  // namespace qm
