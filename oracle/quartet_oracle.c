/*
 * CPU oracle for the Quartet MXFP4 linear-layer hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the arithmetic of the
 * reference's fused Hadamard + MXFP4 pseudo-quantizer and of the GEMMs around it, so the
 * HIP kernels can be checked bit for bit.  Nothing in the product path may link or call it.
 *
 * Reference anchors (paths relative to the reference checkout):
 *   src/models/quantization/quantizers/mxfp4_triton.py:33-174   kernel arithmetic
 *   src/models/quantization/quantizers/mxfp4_triton.py:177-220  wrapper (flat buffer, group 32)
 *   src/models/quantization/quantizers/mxfp4.py:15-34,127-146   kernel flags, STE backward
 *   src/models/quantization/quantizers/mxfp4.py:52-60           sign re-randomisation
 *   src/models/quantization/backward.py:57-85                   operand orientation of the GEMMs
 *   notebooks/benchmark_mxfp4.ipynb (CudaGemm cells)            packed E2M1/E8M0/mask dataflow
 *
 * Canonical choices where the reference is hardware-defined (tensor-core dot order, Triton's
 * approximate log2/exp2/div):
 *   - rotation = fp32 radix-2 Sylvester butterfly, strides 1,2,4,..,hd/2, then ONE multiply by
 *     c = hd^-1/2 rounded to the tensor's dtype, then the column sign;
 *   - group sums (quest) = pairwise tree (adjacent pairs, then pairs of pairs, ...);
 *   - floor(log2 s) = unbiased exponent field; divisions are IEEE round-to-nearest;
 *   - no fused multiply-add anywhere (build with -ffp-contract=off).
 *
 * Parity pins (see tests/): Sylvester matrix vs scipy.linalg.hadamard; order-independent
 * integer fixtures worked out by hand; exhaustive RTN table over all bf16 patterns against the
 * seven strict thresholds; SR bracket/probability grids and unbiasedness; Philox4x32-7 and -10
 * Random123 known-answer vectors; an independent numpy matmul-form restatement (oracle.py);
 * the notebook's recorded error bands.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QO_BF16 0
#define QO_F32 1

#define QO_QUEST_RTN 0
#define QO_ABSMAX_RTN 1
#define QO_ABSMAX_SR 2
#define QO_QUEST_SR 3

/* fl32(2.92247856 / 6.0), mxfp4.py:137 */
static const float QUEST_G = (float)(2.92247856 / 6.0);
/* fl32(1 / 0.75) == fl32(4/3), mxfp4_triton.py:60 */
static const float FOUR_THIRDS = (float)(1.0 / 0.75);

static const float E2M1_VALUE[8] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f};

static inline float bits_to_f32(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static inline uint32_t f32_to_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}
static inline float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }
/* round-to-nearest-even, NaN kept quiet */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t b = f32_to_bits(f);
    if ((b & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((b >> 16) | 0x40);
    b += 0x7fffu + ((b >> 16) & 1u);
    return (uint16_t)(b >> 16);
}

float qo_hadamard_scale(int hd, int dtype) {
    float c = (float)pow((double)hd, -0.5);
    if (dtype == QO_BF16) c = bf16_to_f32(f32_to_bf16(c));
    return c;
}

static inline int sign_is_negative(const uint32_t* sign_bits, int j) {
    return sign_bits ? (int)((sign_bits[j >> 5] >> (j & 31)) & 1u) : 0;
}

/* ---- Philox4x32 (Salmon et al., Random123): the 10-round form and the 7-round form the stream uses ------ */
static void philox4x32(const uint32_t ctr[4], const uint32_t key[2], int rounds, uint32_t out[4]) {
    uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
    uint32_t k0 = key[0], k1 = key[1];
    for (int r = 0; r < rounds; ++r) {
        uint64_t p0 = (uint64_t)0xD2511F53u * c0;
        uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
        uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
        uint32_t n1 = (uint32_t)p1;
        uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
        uint32_t n3 = (uint32_t)p0;
        c0 = n0; c1 = n1; c2 = n2; c3 = n3;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}
void qo_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) { philox4x32(ctr, key, 10, out); }
void qo_philox4x32_7(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) { philox4x32(ctr, key, 7, out); }

/*
 * Uniform for the element at flat offset o of the tensor being quantized (the role of
 * tl.rand(seed, offsets), mxfp4_triton.py:124; the reference's own Philox stream is not reproduced, the
 * contract is equality under identical uniforms).  One Philox4x32-7 call (the fewest rounds Random123
 * publishes as passing its test batteries, and known-answer vectors for) serves sixteen consecutive
 * elements: counter = (o/16 low, o/16 high, 0, 0), key = (seed low, seed high).  Element o reads word
 * (o%16)/4 of the call rotated left by 8 * (o%4) bits and takes its top 22 bits as the field f: every
 * element of a word has its own most significant byte, the bytes below it are shared with the word's
 * other three elements at lower significance, which correlates two of their rounding decisions by less
 * than 2^-8.  The uniform is the largest float below (2^22 - f) / 2^22, so that "u < p" holds exactly
 * when floor(p * 2^22) + f >= 2^22: gfx950's stochastic-rounding convert evaluates this very carry out
 * of a 22-bit addition.  P[round up] = floor(p * 2^22) / 2^22, below p by less than 2^-22.
 */
uint32_t qo_philox_field22(uint64_t seed, uint64_t o) {
    uint32_t ctr[4] = {(uint32_t)(o >> 4), (uint32_t)((o >> 4) >> 32), 0u, 0u};
    uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t w[4];
    philox4x32(ctr, key, 7, w);
    uint32_t word = w[(o & 15) >> 2];
    unsigned s = 8u * (unsigned)(o & 3);
    uint32_t rot = s ? ((word << s) | (word >> (32u - s))) : word;
    return rot >> 10;
}
float qo_philox_uniform(uint64_t seed, uint64_t o) {
    float bound = (float)(4194304u - qo_philox_field22(seed, o)) * (1.0f / 4194304.0f); /* exact: at most 23 significant bits */
    return bits_to_f32(f32_to_bits(bound) - 1u);
}

void qo_philox_uniform_fill(uint64_t seed, int64_t n, float* u) {
    for (int64_t o = 0; o < n; ++o) u[o] = qo_philox_uniform(seed, (uint64_t)o);
}

/* the uniforms of n arbitrary flat offsets (a sample of rows of a large tensor) */
void qo_philox_uniform_at(uint64_t seed, int64_t n, const int64_t* offsets, float* u) {
    for (int64_t i = 0; i < n; ++i) u[i] = qo_philox_uniform(seed, (uint64_t)offsets[i]);
}

/* ---- rotation --------------------------------------------------------------------- */
/* v[0..hd) in place: Sylvester butterfly ascending strides, then * c, then column signs. */
static void rotate_chunk(float* v, int hd, float c, const uint32_t* sign_bits) {
    for (int h = 1; h < hd; h <<= 1) {
        for (int i = 0; i < hd; ++i) {
            if (i & h) continue;
            float a = v[i], b = v[i + h];
            v[i] = a + b;
            v[i + h] = a - b;
        }
    }
    for (int j = 0; j < hd; ++j) {
        float r = v[j] * c;
        v[j] = sign_is_negative(sign_bits, j) ? -r : r;
    }
}

/*
 * Dense rotation of one chunk of 32 (rerotate="O32", mxfp4.py:61-64: H = U V^T of a Gaussian matrix's SVD, applied by
 * tl.dot inside the kernel, mxfp4_triton.py:44-45).  Canonical order: out[j] = fma(v[31], H[31][j], ... fma(v[0],
 * H[0][j], +0)), one fused multiply-add per term in ascending k -- the sequence gfx950's fp32 matrix instruction
 * evaluates.  H holds the matrix already rounded to the tensor's dtype (mxfp4.py:49 casts it).
 */
static void rotate_chunk_dense(float* v, const float* H) {
    float out[32];
    for (int j = 0; j < 32; ++j) {
        float acc = 0.0f;
        for (int k = 0; k < 32; ++k) acc = fmaf(v[k], H[k * 32 + j], acc);
        out[j] = acc;
    }
    memcpy(v, out, sizeof(out));
}

static void round_matrix(const float* matrix, int dtype, float* H) {
    for (int i = 0; i < 1024; ++i) H[i] = dtype == QO_BF16 ? bf16_to_f32(f32_to_bf16(matrix[i])) : matrix[i];
}

static float tree_sum32(const float* p) {
    float t[32];
    memcpy(t, p, sizeof(t));
    for (int n = 16; n >= 1; n >>= 1)
        for (int i = 0; i < n; ++i) t[i] = t[2 * i] + t[2 * i + 1];
    return t[0];
}

static inline int floor_log2_f32(float s) { /* s finite, > 0 */
    int e;
    frexpf(s, &e); /* s = m * 2^e, m in [0.5,1) */
    return e - 1;
}

static inline int clamp_int(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

/* RTN onto the E2M1 magnitude grid, strict thresholds, mxfp4_triton.py:131-159 */
static inline int rtn_code(float A) {
    if (A > 5.0f) return 7;
    if (A > 3.5f) return 6;
    if (A > 2.5f) return 5;
    if (A > 1.75f) return 4;
    if (A > 1.25f) return 3;
    if (A > 0.75f) return 2;
    if (A > 0.25f) return 1;
    return 0;
}

/* SR, mxfp4_triton.py:70-129: bracket by strict '>', p = (A-lo)/(hi-lo), up iff u < p */
static inline int sr_code(float A, float u) {
    int lo;
    if (A > 4.0f) lo = 6;
    else if (A > 3.0f) lo = 5;
    else if (A > 2.0f) lo = 4;
    else if (A > 1.5f) lo = 3;
    else if (A > 1.0f) lo = 2;
    else if (A > 0.5f) lo = 1;
    else lo = 0;
    float vlo = E2M1_VALUE[lo], vhi = E2M1_VALUE[lo + 1];
    float p = (A - vlo) / (vhi - vlo);
    return (u < p) ? lo + 1 : lo;
}

/*
 * Quantize one MX group of 32 rotated values g.  Writes 32 nibble codes (unpacked, one per
 * byte), the E8M0 byte, 32 mask flags and the 32 dequantized fp32 values.
 */
static void quantize_group(const float* g, int mode, const float* u, uint8_t* code, uint8_t* e8m0,
                           uint8_t* keep, float* deq) {
    float t[32];
    float scale; /* what the dequantized value is multiplied by */
    int quest = (mode == QO_QUEST_RTN || mode == QO_QUEST_SR);
    int sr = (mode == QO_ABSMAX_SR || mode == QO_QUEST_SR);
    if (quest) {
        float sq[32];
        for (int i = 0; i < 32; ++i) sq[i] = g[i] * g[i];
        float ms = tree_sum32(sq) * 0.03125f;
        float m = tree_sum32(g) * 0.03125f;
        float mm = m * m;
        float var = ms - mm;
        if (!(var > 0.0f)) var = 0.0f; /* reference gives NaN for var<0; clamp instead */
        float sd = sqrtf(var);
        float gs = QUEST_G * sd;
        float s = gs + 1e-8f;
        /* floor(log2 s): s >= 1e-8 is a normal number, so this is its exponent field; an
           infinite or NaN s reads as 128 and clamps to 127 */
        int E = clamp_int((int)((f32_to_bits(s) >> 23) & 0xffu) - 127, -127, 127);
        *e8m0 = (uint8_t)(E + 127);
        scale = ldexpf(1.0f, E);
        for (int i = 0; i < 32; ++i) t[i] = ldexpf(g[i], -E);
    } else {
        float a = 0.0f;
        int has_nan = 0;
        for (int i = 0; i < 32; ++i) {
            float v = fabsf(g[i]);
            if (v != v) has_nan = 1;
            if (v > a) a = v;
        }
        if (a == 0.0f || has_nan || isinf(a)) {
            /* log2(0) = -inf in the reference: scale 0, t = NaN, every compare false -> -0 */
            *e8m0 = (a == 0.0f && !has_nan) ? 0 : 254;
            for (int i = 0; i < 32; ++i) {
                code[i] = 0x8;
                keep[i] = 0;
                deq[i] = -0.0f;
            }
            return;
        }
        int k = clamp_int(floor_log2_f32(a) - 2, -127, 127);
        *e8m0 = (uint8_t)(k + 127);
        scale = ldexpf(FOUR_THIRDS, k);
        for (int i = 0; i < 32; ++i) t[i] = ldexpf(g[i], -k) / FOUR_THIRDS;
    }
    for (int i = 0; i < 32; ++i) {
        float A = fabsf(t[i]);
        /* sign = "not (t > 0)" (mxfp4_triton.py:65-69); t and g have the same sign, and taking it
           from g keeps it defined when t underflows */
        int neg = !(g[i] > 0.0f);
        int mag = sr ? sr_code(A, u[i]) : rtn_code(A);
        code[i] = (uint8_t)(mag | (neg << 3));
        keep[i] = (uint8_t)(A < 6.0f);
        float q = E2M1_VALUE[mag];
        deq[i] = (neg ? -q : q) * scale;
    }
}

static inline float load_elem(const void* x, int dtype, int64_t idx) {
    return dtype == QO_BF16 ? bf16_to_f32(((const uint16_t*)x)[idx]) : ((const float*)x)[idx];
}
static inline void store_elem(void* y, int dtype, int64_t idx, float v) {
    if (dtype == QO_BF16) ((uint16_t*)y)[idx] = f32_to_bf16(v);
    else ((float*)y)[idx] = v;
}

/* shared tail: rotate a logical row already converted to fp32, quantize its groups, emit */
static void quantize_row(float* row, int64_t r, int64_t cols, int hd, float c,
                         const uint32_t* sign_bits, int mode, const float* u, uint64_t seed,
                         uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                         int out_dtype, float* rotated, const float* dense) {
    if (dense) {
        for (int64_t j0 = 0; j0 < cols; j0 += 32) rotate_chunk_dense(row + j0, dense);
    } else {
        for (int64_t j0 = 0; j0 < cols; j0 += hd) rotate_chunk(row + j0, hd, c, sign_bits);
    }
    if (rotated) memcpy(rotated + r * cols, row, (size_t)cols * sizeof(float));
    for (int64_t j0 = 0; j0 < cols; j0 += 32) {
        uint8_t code[32], keep[32], e8;
        float deq[32], ug[32];
        int sr = (mode == QO_ABSMAX_SR || mode == QO_QUEST_SR);
        if (sr) {
            for (int i = 0; i < 32; ++i)
                ug[i] = u ? u[r * cols + j0 + i] : qo_philox_uniform(seed, (uint64_t)(r * cols + j0 + i));
        }
        quantize_group(row + j0, mode, ug, code, &e8, keep, deq);
        scales[r * (cols / 32) + j0 / 32] = e8;
        for (int i = 0; i < 16; ++i)
            codes[r * (cols / 2) + j0 / 2 + i] = (uint8_t)(code[2 * i] | (code[2 * i + 1] << 4));
        if (maskbits) {
            for (int b = 0; b < 4; ++b) {
                uint8_t m = 0;
                for (int i = 0; i < 8; ++i) m |= (uint8_t)(keep[8 * b + i] << i);
                maskbits[r * (cols / 8) + j0 / 8 + b] = m;
            }
        }
        if (dequant)
            for (int i = 0; i < 32; ++i) store_elem(dequant, out_dtype, r * cols + j0 + i, deq[i]);
    }
}

/*
 * Fused rotate + MXFP4 quantize of a logical [rows, cols] tensor along cols.
 * transposed_in != 0: x is stored as [cols, rows] row-major (the logical tensor is its
 * transpose; backward.py:73,81-82 do this with .T.contiguous()).
 * u: explicit uniforms indexed by logical flat offset, or NULL for the Philox stream of seed.
 */
static int quantize_core(const void* x, int dtype, int64_t rows, int64_t cols, int hd,
                         const uint32_t* sign_bits, int mode, int transposed_in, const float* u,
                         uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                         float* rotated, const float* dense) {
    /* hd == 1: the input is already rotated (a dense rotation applied by the caller, mxfp4.py:61-64): the butterfly
       has no stage and c = 1 */
    if (!(hd == 1 || hd == 32 || hd == 64 || hd == 128) || cols % hd || cols % 32 || rows < 0 || cols < 0) return -1;
    if (mode < 0 || mode > 3 || (dtype != QO_BF16 && dtype != QO_F32)) return -1;
    float c = qo_hadamard_scale(hd, dtype);
    int err = 0;
#pragma omp parallel
    {
        float* row = (float*)malloc((size_t)(cols ? cols : 1) * sizeof(float));
        if (!row) {
#pragma omp atomic write
            err = 1;
        }
#pragma omp for schedule(static)
        for (int64_t r = 0; r < rows; ++r) {
            if (!row) continue;
            for (int64_t j = 0; j < cols; ++j)
                row[j] = load_elem(x, dtype, transposed_in ? j * rows + r : r * cols + j);
            quantize_row(row, r, cols, hd, c, sign_bits, mode, u, seed, codes, scales, maskbits,
                         dequant, dtype, rotated, dense);
        }
        free(row);
    }
    return err ? -2 : 0;
}

int qo_quantize(const void* x, int dtype, int64_t rows, int64_t cols, int hd,
                const uint32_t* sign_bits, int mode, int transposed_in, const float* u,
                uint64_t seed, uint8_t* codes, uint8_t* scales, uint8_t* maskbits, void* dequant,
                float* rotated) {
    return quantize_core(x, dtype, rows, cols, hd, sign_bits, mode, transposed_in, u, seed, codes, scales,
                         maskbits, dequant, rotated, NULL);
}

/* the same with a dense 32x32 rotation: matrix [32][32] fp32 row-major (H[k][j]), rounded to dtype here */
int qo_quantize_dense(const void* x, int dtype, int64_t rows, int64_t cols, const float* matrix, int mode,
                      int transposed_in, const float* u, uint64_t seed, uint8_t* codes, uint8_t* scales,
                      uint8_t* maskbits, void* dequant, float* rotated) {
    float H[1024];
    if (!matrix || (dtype != QO_BF16 && dtype != QO_F32)) return -1;
    round_matrix(matrix, dtype, H);
    return quantize_core(x, dtype, rows, cols, 32, NULL, mode, transposed_in, u, seed, codes, scales, maskbits,
                         dequant, rotated, H);
}

/* value of a packed MXFP4 element; post = 1 (quest coding) or fl32(4/3) (absmax coding) */
static inline float mx_value(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C,
                             int64_t r, int64_t c, float post) {
    (void)R;
    uint8_t byte = codes[r * (C / 2) + c / 2];
    uint8_t nib = (c & 1) ? (byte >> 4) : (byte & 15);
    float q = E2M1_VALUE[nib & 7];
    if (nib & 8) q = -q;
    float scale = ldexpf(post, (int)scales[r * (C / 32) + c / 32] - 127);
    return q * scale;
}

int qo_dequantize(const uint8_t* codes, const uint8_t* scales, int64_t R, int64_t C, float post,
                  void* out, int out_dtype) {
    if (C % 32) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < R; ++r)
        for (int64_t c = 0; c < C; ++c)
            store_elem(out, out_dtype, r * C + c, mx_value(codes, scales, R, C, r, c, post));
    return 0;
}

/*
 * Dequantize a packed [R, C] MXFP4 tensor (values rounded to val_dtype, as the reference keeps
 * its pseudo-quantized tensors in the input dtype), transpose, rotate and re-quantize along R:
 * outputs codes_out [C, R/2], scales_out [C, R/32].  backward.py:73,82 (.T.contiguous() of the
 * saved quantized operand, then g_quantizer).
 */
static int requantize_core(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R,
                           int64_t C, float post, int val_dtype, int hd,
                           const uint32_t* sign_bits, int mode, const float* u, uint64_t seed,
                           uint8_t* codes_out, uint8_t* scales_out, void* dequant,
                           float* rotated, const float* dense) {
    if (!(hd == 32 || hd == 64 || hd == 128) || R % hd || C % 32) return -1;
    float c = qo_hadamard_scale(hd, val_dtype);
    int err = 0;
#pragma omp parallel
    {
        float* row = (float*)malloc((size_t)(R ? R : 1) * sizeof(float));
        if (!row) {
#pragma omp atomic write
            err = 1;
        }
#pragma omp for schedule(static)
        for (int64_t j = 0; j < C; ++j) {
            if (!row) continue;
            for (int64_t r = 0; r < R; ++r) {
                float v = mx_value(codes_in, scales_in, R, C, r, j, post);
                if (val_dtype == QO_BF16) v = bf16_to_f32(f32_to_bf16(v));
                row[r] = v;
            }
            quantize_row(row, j, R, hd, c, sign_bits, mode, u, seed, codes_out, scales_out, NULL,
                         dequant, val_dtype, rotated, dense);
        }
        free(row);
    }
    return err ? -2 : 0;
}

int qo_requantize_transposed(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R,
                             int64_t C, float post, int val_dtype, int hd,
                             const uint32_t* sign_bits, int mode, const float* u, uint64_t seed,
                             uint8_t* codes_out, uint8_t* scales_out, void* dequant,
                             float* rotated) {
    return requantize_core(codes_in, scales_in, R, C, post, val_dtype, hd, sign_bits, mode, u, seed, codes_out,
                           scales_out, dequant, rotated, NULL);
}

int qo_requantize_transposed_dense(const uint8_t* codes_in, const uint8_t* scales_in, int64_t R, int64_t C,
                                   float post, int val_dtype, const float* matrix, int mode, const float* u,
                                   uint64_t seed, uint8_t* codes_out, uint8_t* scales_out, void* dequant,
                                   float* rotated) {
    float H[1024];
    if (!matrix || (val_dtype != QO_BF16 && val_dtype != QO_F32)) return -1;
    round_matrix(matrix, val_dtype, H);
    return requantize_core(codes_in, scales_in, R, C, post, val_dtype, 32, NULL, mode, u, seed, codes_out,
                           scales_out, dequant, rotated, H);
}

/*
 * C[m,n] = alpha * sum_k a[m,k] * b[n,k] on the dequantized operands ("TN": both operands
 * row-major with K contiguous; backward.py:62,71-75,79-83).  fp64 accumulation; posts are the
 * per-operand constants (1 or fl32(4/3)) folded into each element in fp32 first.
 */
int qo_gemm_tn(const uint8_t* a_codes, const uint8_t* a_scales, float a_post,
               const uint8_t* b_codes, const uint8_t* b_scales, float b_post, int64_t M, int64_t N,
               int64_t K, double alpha, double* C) {
    if (K % 32) return -1;
    float* A = (float*)malloc((size_t)(M * K > 0 ? M * K : 1) * sizeof(float));
    float* B = (float*)malloc((size_t)(N * K > 0 ? N * K : 1) * sizeof(float));
    if (!A || !B) {
        free(A);
        free(B);
        return -2;
    }
    qo_dequantize(a_codes, a_scales, M, K, a_post, A, QO_F32);
    qo_dequantize(b_codes, b_scales, N, K, b_post, B, QO_F32);
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            const float* a = A + m * K;
            const float* b = B + n * K;
            double s = 0.0;
            for (int64_t k = 0; k < K; ++k) s += (double)a[k] * (double)b[k];
            C[m * N + n] = alpha * s;
        }
    }
    free(A);
    free(B);
    return 0;
}

/*
 * Straight-through backward of the forward quantizer, mxfp4.py:143-146:
 * out = ((g * mask).view(-1, hd)) @ H^T with H = c * S * diag(signs).  Signs hit the input
 * column, then the butterfly, then c.  maskbits may be NULL (mxfp4.py:31-34: no mask).
 */
int qo_masked_hadamard_bwd(const void* g, int g_dtype, int64_t rows, int64_t cols, int hd,
                           int scale_dtype, const uint32_t* sign_bits, const uint8_t* maskbits,
                           void* out, int out_dtype) {
    if (!(hd == 32 || hd == 64 || hd == 128) || cols % hd) return -1;
    float c = qo_hadamard_scale(hd, scale_dtype);
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        float v[128];
        for (int64_t j0 = 0; j0 < cols; j0 += hd) {
            for (int j = 0; j < hd; ++j) {
                int64_t idx = r * cols + j0 + j;
                float x = load_elem(g, g_dtype, idx);
                if (maskbits && !((maskbits[idx >> 3] >> (idx & 7)) & 1)) x = 0.0f * x;
                v[j] = sign_is_negative(sign_bits, j) ? -x : x;
            }
            for (int h = 1; h < hd; h <<= 1)
                for (int i = 0; i < hd; ++i) {
                    if (i & h) continue;
                    float a = v[i], b = v[i + h];
                    v[i] = a + b;
                    v[i + h] = a - b;
                }
            for (int j = 0; j < hd; ++j) store_elem(out, out_dtype, r * cols + j0 + j, v[j] * c);
        }
    }
    return 0;
}

/*
 * Producers in front of the activation quantizer (the callers' side of the path):
 *   RMSNorm  src/models/llama.py:64-75   (x.float() * rsqrt(mean(x^2) + eps)).type_as(x) * weight
 *   SwiGLU   src/models/llama.py:113-114 silu(up) * gate, with (up, gate) = split of the fused w12 output
 * torch's reductions and its device exp are implementation-defined; the canonical choices here:
 *   - sum of squares of a row: sixteen interleaved partial sums (partial j takes groups j, j+16, j+32, ... of 32
 *     consecutive elements, each group summed by the pairwise tree, added in ascending order), then the pairwise tree
 *     over the sixteen partials; mean = sum / cols, factor = 1 / sqrt(mean + eps), IEEE divisions and square root;
 *   - e^z = 2^n * P(r): n = rint(z * fl32(log2 e)), r = fma(n, -ln2_lo, fma(n, -ln2_hi, z)), P = degree-7 Taylor
 *     polynomial evaluated by Horner's rule in fmas; silu(x) = x / (1 + e^-x);
 *   - with a bf16 tensor every torch op rounds its result to bf16: silu, then the product.
 * Pins: tests compare qo_exp with the C library's double-precision exp (<= 1.5 ulp), qo_silu and qo_rmsnorm with
 * float64 evaluations of the reference's formulas, and closed forms (constant rows, zeros, saturation).
 */
float qo_exp(float z) {
    if (z != z) return z;
    if (z > 88.72283935546875f) return INFINITY;
    if (z < -104.0f) return 0.0f;
    const float n = rintf(z * 1.44269502162933349609375f);
    float r = fmaf(n, -0.693145751953125f, z);
    r = fmaf(n, -1.428606765330187045037746429443359375e-06f, r);
    float p = 1.0f / 5040.0f;
    const float coef[7] = {1.0f / 720.0f, 1.0f / 120.0f, 1.0f / 24.0f, 1.0f / 6.0f, 0.5f, 1.0f, 1.0f};
    for (int i = 0; i < 7; ++i) p = fmaf(p, r, coef[i]);
    return ldexpf(p, (int)n);
}

float qo_silu(float x) { return x / (1.0f + qo_exp(-x)); }

/* out [rows, cols] fp32 = what RMSNorm hands to the linear layer; factor [rows] = the per-row 1/sqrt(mean + eps) */
int qo_rmsnorm(const void* x, int dtype, const float* gain, float eps, int64_t rows, int64_t cols, float* out,
               float* factor) {
    if (cols % 32 || rows < 0 || cols <= 0 || (dtype != QO_BF16 && dtype != QO_F32)) return -1;
    const int64_t groups = cols / 32;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        float partial[16];
        for (int j = 0; j < 16; ++j) {
            float acc = 0.0f;
            for (int64_t g = j; g < groups; g += 16) {
                float sq[32];
                for (int i = 0; i < 32; ++i) {
                    const float v = load_elem(x, dtype, r * cols + g * 32 + i);
                    sq[i] = v * v;
                }
                acc = acc + tree_sum32(sq);
            }
            partial[j] = acc;
        }
        for (int n = 8; n >= 1; n >>= 1)
            for (int i = 0; i < n; ++i) partial[i] = partial[2 * i] + partial[2 * i + 1];
        const float f = 1.0f / sqrtf(partial[0] / (float)cols + eps);
        if (factor) factor[r] = f;
        for (int64_t j = 0; j < cols; ++j) {
            float n = load_elem(x, dtype, r * cols + j) * f;
            if (dtype == QO_BF16) n = bf16_to_f32(f32_to_bf16(n)); /* .type_as(x) */
            out[r * cols + j] = n * gain[j];
        }
    }
    return 0;
}

/* out [rows, hidden] of h12's dtype = silu(h12[:, :hidden]) * h12[:, hidden:] */
int qo_swiglu(const void* h12, int dtype, int64_t rows, int64_t hidden, void* out) {
    if (rows < 0 || hidden <= 0 || (dtype != QO_BF16 && dtype != QO_F32)) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        for (int64_t j = 0; j < hidden; ++j) {
            const float up = load_elem(h12, dtype, r * 2 * hidden + j);
            const float gate = load_elem(h12, dtype, r * 2 * hidden + hidden + j);
            float a = qo_silu(up);
            if (dtype == QO_BF16) a = bf16_to_f32(f32_to_bf16(a));
            store_elem(out, dtype, r * hidden + j, a * gate);
        }
    }
    return 0;
}

/* single-value helpers exported for exhaustive table tests */
int qo_rtn_code(float A) { return rtn_code(A); }
int qo_sr_code(float A, float u) { return sr_code(A, u); }
float qo_div_four_thirds(float g) { return g / FOUR_THIRDS; }
