// Rotary position embedding of the fused attention projection, in the model the quantized linears sit in
// (src/models/llama.py:43-61 of the reference: consecutive element pairs (2i, 2i+1) of every head of q and k are
// rotated by position * theta^(-2i/head_dim), evaluated in fp32).  One pass splits the c_attn output
// [rows, 3C] = (q, k, v) into three [rows, C] tensors, q and k rotated; the backward pass merges the three
// gradients back into [rows, 3C] with the inverse rotation.  Arithmetic as the reference's torch ops perform it:
// every product and every sum rounded to fp32, no fused multiply-add.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "qm_kernels.h"
#include "qm_math.h"

namespace qm {

namespace {

typedef float v2f __attribute__((ext_vector_type(2)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

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
        const float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
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
        reinterpret_cast<float4*>(p)[0] = make_float4(v[0], v[1], v[2], v[3]);
        reinterpret_cast<float4*>(p)[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
}

// One lane per 8 consecutive elements of the [rows, 3C] side.  INVERSE = false: fused -> (q, k, v);
// INVERSE = true: (dq, dk, dv) -> fused, rotation by the negative angle.
template <typename TFused, typename TPart, bool INVERSE>
__global__ __launch_bounds__(256) void rope_qkv_kernel(TFused* __restrict__ fused, TPart* __restrict__ q, TPart* __restrict__ k,
                                                       TPart* __restrict__ v, const float* __restrict__ table, int64_t rows,
                                                       int seq_len, int C, int head_dim) {
    const int octets_per_row = 3 * C / 8;
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= rows * octets_per_row) return;
    const int64_t row = o / octets_per_row;
    const int col = (int)(o - row * octets_per_row) * 8;
    const int part = col / C, c = col - part * C;
    TPart* part_ptr = (part == 0 ? q : (part == 1 ? k : v)) + row * C + c;
    TFused* fused_ptr = fused + row * 3 * C + col;
    float x[8];
    if constexpr (INVERSE) load8<TPart>(part_ptr, x);
    else load8<TFused>(fused_ptr, x);
    if (part < 2) {
        const int pos = (int)(row % seq_len), pair = (c % head_dim) >> 1;
        float cs[8];  // (cos, sin) of the four pairs
        load8<float>(table + ((int64_t)pos * (head_dim / 2) + pair) * 2, cs);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float a = x[2 * i], b = x[2 * i + 1], co = cs[2 * i], si = cs[2 * i + 1];
            if constexpr (INVERSE) {
                x[2 * i] = a * co + b * si;
                x[2 * i + 1] = b * co - a * si;
            } else {
                x[2 * i] = a * co - b * si;
                x[2 * i + 1] = a * si + b * co;
            }
        }
    }
    if constexpr (INVERSE) store8<TFused>(fused_ptr, x);
    else store8<TPart>(part_ptr, x);
}

template <bool INVERSE>
void launch_rope(void* fused, int fused_dtype, void* q, void* k, void* v, int part_dtype, const float* table, int64_t rows,
                 int seq_len, int C, int head_dim, hipStream_t stream) {
    const dim3 grid((unsigned)((rows * (3 * C / 8) + 255) / 256)), block(256);
#define QM_ROPE(TF, TP)                                                                                                 \
    rope_qkv_kernel<TF, TP, INVERSE><<<grid, block, 0, stream>>>(reinterpret_cast<TF*>(fused), reinterpret_cast<TP*>(q), \
                                                                 reinterpret_cast<TP*>(k), reinterpret_cast<TP*>(v), table, \
                                                                 rows, seq_len, C, head_dim)
    if (fused_dtype == BF16 && part_dtype == BF16) QM_ROPE(uint16_t, uint16_t);
    else if (fused_dtype == BF16) QM_ROPE(uint16_t, float);
    else if (part_dtype == BF16) QM_ROPE(float, uint16_t);
    else QM_ROPE(float, float);
#undef QM_ROPE
}

}  // namespace

// C % 8 == 0, head_dim % 8 == 0, C % head_dim == 0; table [seq_len, head_dim / 2, 2] fp32 = (cos, sin); row r of the
// tensors sits at position r % seq_len
hipError_t rope_split_qkv(const void* qkv, int qkv_dtype, int64_t rows, int seq_len, int C, int head_dim, const float* table,
                          void* q, void* k, void* v, int out_dtype, hipStream_t stream) {
    if (rows == 0 || C == 0) return hipSuccess;
    launch_rope<false>(const_cast<void*>(qkv), qkv_dtype, q, k, v, out_dtype, table, rows, seq_len, C, head_dim, stream);
    return hipGetLastError();
}

hipError_t rope_merge_qkv_grad(const void* dq, const void* dk, const void* dv, int grad_dtype, int64_t rows, int seq_len, int C,
                               int head_dim, const float* table, void* d_qkv, int out_dtype, hipStream_t stream) {
    if (rows == 0 || C == 0) return hipSuccess;
    launch_rope<true>(d_qkv, out_dtype, const_cast<void*>(dq), const_cast<void*>(dk), const_cast<void*>(dv), grad_dtype, table, rows,
                      seq_len, C, head_dim, stream);
    return hipGetLastError();
}

}  // namespace qm
