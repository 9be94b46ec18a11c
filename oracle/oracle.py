"""CPU oracle for the Quartet MXFP4 hot path -- TEST INFRASTRUCTURE ONLY.

Two independent restatements of the reference's arithmetic
(src/models/quantization/quantizers/mxfp4_triton.py:33-174):

* the C library ``quartet_oracle.c`` (canonical butterfly order, bit-exact target for the HIP
  kernels), loaded here through ctypes;
* ``np_*`` functions: a numpy matmul-form restatement (dense ``x @ H`` in float64, library
  ``std``/``max``, bucketised rounding) used only to pin the C code -- a transposed operand, a
  dropped term or a wrong tie direction in either one shows up as a disagreement.

Only tests, ``__graft_entry__.smoke()`` and ``bench.py``'s cpu_baseline leg may import this.
Arrays: bf16 tensors travel as ``uint16`` numpy arrays, fp32 as ``float32``.
"""
import ctypes
import os
import subprocess

import numpy as np

QUEST_RTN, ABSMAX_RTN, ABSMAX_SR, QUEST_SR = 0, 1, 2, 3
BF16, F32 = 0, 1

E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0], dtype=np.float32)
FOUR_THIRDS = np.float32(1.0 / 0.75)
QUEST_G = np.float32(2.92247856 / 6.0)

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libquartet_oracle.so")
_lib = None


def build(force=False):
    """Compile quartet_oracle.c with the committed Makefile."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i32, i64, u64, f32, f64 = (ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                       ctypes.c_uint64, ctypes.c_float, ctypes.c_double)
        L.qo_hadamard_scale.restype = f32
        L.qo_hadamard_scale.argtypes = [i32, i32]
        L.qo_philox4x32_10.argtypes = [vp, vp, vp]
        L.qo_philox4x32_7.argtypes = [vp, vp, vp]
        L.qo_philox_field22.restype = ctypes.c_uint32
        L.qo_philox_field22.argtypes = [u64, u64]
        L.qo_philox_uniform.restype = f32
        L.qo_philox_uniform.argtypes = [u64, u64]
        L.qo_philox_uniform_fill.argtypes = [u64, i64, vp]
        L.qo_philox_uniform_at.argtypes = [u64, i64, vp, vp]
        L.qo_quantize.restype = i32
        L.qo_quantize.argtypes = [vp, i32, i64, i64, i32, vp, i32, i32, vp, u64, vp, vp, vp, vp, vp]
        L.qo_quantize_dense.restype = i32
        L.qo_quantize_dense.argtypes = [vp, i32, i64, i64, vp, i32, i32, vp, u64, vp, vp, vp, vp, vp]
        L.qo_requantize_transposed_dense.restype = i32
        L.qo_requantize_transposed_dense.argtypes = [vp, vp, i64, i64, f32, i32, vp, i32, vp, u64, vp, vp, vp, vp]
        L.qo_dequantize.restype = i32
        L.qo_dequantize.argtypes = [vp, vp, i64, i64, f32, vp, i32]
        L.qo_requantize_transposed.restype = i32
        L.qo_requantize_transposed.argtypes = [vp, vp, i64, i64, f32, i32, i32, vp, i32, vp, u64,
                                               vp, vp, vp, vp]
        L.qo_gemm_tn.restype = i32
        L.qo_gemm_tn.argtypes = [vp, vp, f32, vp, vp, f32, i64, i64, i64, f64, vp]
        L.qo_masked_hadamard_bwd.restype = i32
        L.qo_masked_hadamard_bwd.argtypes = [vp, i32, i64, i64, i32, i32, vp, vp, vp, i32]
        L.qo_rtn_code.restype = i32
        L.qo_rtn_code.argtypes = [f32]
        L.qo_sr_code.restype = i32
        L.qo_sr_code.argtypes = [f32, f32]
        L.qo_div_four_thirds.restype = f32
        L.qo_div_four_thirds.argtypes = [f32]
        L.qo_exp.restype = f32
        L.qo_exp.argtypes = [f32]
        L.qo_silu.restype = f32
        L.qo_silu.argtypes = [f32]
        L.qo_rmsnorm.restype = i32
        L.qo_rmsnorm.argtypes = [vp, i32, vp, f32, i64, i64, vp, vp]
        L.qo_swiglu.restype = i32
        L.qo_swiglu.argtypes = [vp, i32, i64, i64, vp]
        _lib = L
    return _lib


# ---------------------------------------------------------------------------------------------
# dtype helpers
# ---------------------------------------------------------------------------------------------
def f32_to_bf16_bits(x):
    """float32 array -> uint16 bf16 bit patterns, round-to-nearest-even."""
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (b & 0x7FFFFFFF) > 0x7F800000
    r = ((b + (0x7FFF + ((b >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((b[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_bits_to_f32(h):
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def _dtype_of(x):
    if x.dtype == np.uint16:
        return BF16
    if x.dtype == np.float32:
        return F32
    raise TypeError("oracle arrays are uint16 (bf16 bits) or float32")


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def sign_bits_from_signs(signs):
    """signs: iterable of +1/-1 of length hd -> uint32[4] bit mask (bit j set = column j negated)."""
    out = np.zeros(4, dtype=np.uint32)
    if signs is None:
        return None
    for j, s in enumerate(np.asarray(signs).tolist()):
        if s < 0:
            out[j >> 5] |= np.uint32(1 << (j & 31))
    return out


def hadamard_scale(hd, dtype):
    return np.float32(lib().qo_hadamard_scale(hd, dtype))


# ---------------------------------------------------------------------------------------------
# ctypes wrappers around the canonical C oracle
# ---------------------------------------------------------------------------------------------
def philox4x32(ctr, key, rounds=7):
    """Philox4x32 with 7 rounds (what the stochastic-rounding stream uses) or 10."""
    c = np.asarray(ctr, dtype=np.uint32)
    k = np.asarray(key, dtype=np.uint32)
    o = np.zeros(4, dtype=np.uint32)
    {7: lib().qo_philox4x32_7, 10: lib().qo_philox4x32_10}[rounds](_ptr(c), _ptr(k), _ptr(o))
    return o


def philox_field22(seed, o):
    """The 22-bit random field of the element at flat offset o."""
    return int(lib().qo_philox_field22(seed, o))


def philox_uniform(seed, n):
    """The stream's uniforms of flat element offsets 0..n-1."""
    u = np.empty(n, dtype=np.float32)
    lib().qo_philox_uniform_fill(seed, n, _ptr(u))
    return u


def philox_uniform_at(seed, offsets):
    """The stream's uniforms at the given flat element offsets (any shape of int64), same shape back."""
    off = np.ascontiguousarray(offsets, dtype=np.int64)
    u = np.empty(off.shape, dtype=np.float32)
    lib().qo_philox_uniform_at(seed, off.size, _ptr(off), _ptr(u))
    return u


def quantize(x, hd=32, signs=None, mode=QUEST_RTN, transposed_in=False, u=None, seed=0,
             want_mask=False, want_dequant=False, want_rotated=False, matrix=None):
    """Returns dict(codes [R,C/2] u8, scales [R,C/32] u8, mask [R,C/8] u8|None,
    dequant like logical x|None, rotated f32|None).  Logical shape is x.shape, or its transpose
    when transposed_in.  `matrix` (float32 [32, 32]): a dense rotation replaces the Hadamard block
    (hd and signs are then unused); it is rounded to x's dtype first."""
    x = np.ascontiguousarray(x)
    dt = _dtype_of(x)
    rows, cols = (x.shape[1], x.shape[0]) if transposed_in else x.shape
    sb = sign_bits_from_signs(signs)
    codes = np.empty((rows, cols // 2), dtype=np.uint8)
    scales = np.empty((rows, cols // 32), dtype=np.uint8)
    mask = np.empty((rows, cols // 8), dtype=np.uint8) if want_mask else None
    deq = np.empty((rows, cols), dtype=x.dtype) if want_dequant else None
    rot = np.empty((rows, cols), dtype=np.float32) if want_rotated else None
    if u is not None:
        u = np.ascontiguousarray(u, dtype=np.float32)
        assert u.size == rows * cols
    if matrix is not None:
        m = np.ascontiguousarray(matrix, dtype=np.float32)
        assert m.shape == (32, 32)
        rc = lib().qo_quantize_dense(_ptr(x), dt, rows, cols, _ptr(m), mode, int(transposed_in), _ptr(u), seed,
                                     _ptr(codes), _ptr(scales), _ptr(mask), _ptr(deq), _ptr(rot))
    else:
        rc = lib().qo_quantize(_ptr(x), dt, rows, cols, hd, _ptr(sb), mode, int(transposed_in),
                               _ptr(u), seed, _ptr(codes), _ptr(scales), _ptr(mask), _ptr(deq),
                               _ptr(rot))
    if rc != 0:
        raise ValueError(f"qo_quantize rejected its arguments (rc={rc})")
    return dict(codes=codes, scales=scales, mask=mask, dequant=deq, rotated=rot)


def dequantize(codes, scales, post=1.0, out_dtype=F32):
    R, C = codes.shape[0], codes.shape[1] * 2
    out = np.empty((R, C), dtype=np.float32 if out_dtype == F32 else np.uint16)
    rc = lib().qo_dequantize(_ptr(np.ascontiguousarray(codes)), _ptr(np.ascontiguousarray(scales)),
                             R, C, post, _ptr(out), out_dtype)
    if rc != 0:
        raise ValueError(f"qo_dequantize rc={rc}")
    return out


def requantize_transposed(codes, scales, post=1.0, val_dtype=BF16, hd=32, signs=None,
                          mode=ABSMAX_SR, u=None, seed=0, want_dequant=False, want_rotated=False, matrix=None):
    R, C = codes.shape[0], codes.shape[1] * 2
    sb = sign_bits_from_signs(signs)
    codes_out = np.empty((C, R // 2), dtype=np.uint8)
    scales_out = np.empty((C, R // 32), dtype=np.uint8)
    deq = np.empty((C, R), dtype=np.uint16 if val_dtype == BF16 else np.float32) if want_dequant else None
    rot = np.empty((C, R), dtype=np.float32) if want_rotated else None
    if u is not None:
        u = np.ascontiguousarray(u, dtype=np.float32)
        assert u.size == R * C
    if matrix is not None:
        m = np.ascontiguousarray(matrix, dtype=np.float32)
        assert m.shape == (32, 32)
        rc = lib().qo_requantize_transposed_dense(_ptr(np.ascontiguousarray(codes)), _ptr(np.ascontiguousarray(scales)),
                                                  R, C, post, val_dtype, _ptr(m), mode, _ptr(u), seed, _ptr(codes_out),
                                                  _ptr(scales_out), _ptr(deq), _ptr(rot))
    else:
        rc = lib().qo_requantize_transposed(_ptr(np.ascontiguousarray(codes)),
                                            _ptr(np.ascontiguousarray(scales)), R, C, post, val_dtype,
                                            hd, _ptr(sb), mode, _ptr(u), seed, _ptr(codes_out),
                                            _ptr(scales_out), _ptr(deq), _ptr(rot))
    if rc != 0:
        raise ValueError(f"qo_requantize_transposed rc={rc}")
    return dict(codes=codes_out, scales=scales_out, dequant=deq, rotated=rot)


def gemm_tn(a_codes, a_scales, b_codes, b_scales, alpha=1.0, a_post=1.0, b_post=1.0):
    M, K = a_codes.shape[0], a_codes.shape[1] * 2
    N = b_codes.shape[0]
    assert b_codes.shape[1] * 2 == K
    C = np.empty((M, N), dtype=np.float64)
    rc = lib().qo_gemm_tn(_ptr(np.ascontiguousarray(a_codes)), _ptr(np.ascontiguousarray(a_scales)),
                          a_post, _ptr(np.ascontiguousarray(b_codes)),
                          _ptr(np.ascontiguousarray(b_scales)), b_post, M, N, K, alpha, _ptr(C))
    if rc != 0:
        raise ValueError(f"qo_gemm_tn rc={rc}")
    return C


def masked_hadamard_bwd(g, hd=32, scale_dtype=BF16, signs=None, maskbits=None, out_dtype=None):
    g = np.ascontiguousarray(g)
    dt = _dtype_of(g)
    out_dtype = dt if out_dtype is None else out_dtype
    rows, cols = g.shape
    out = np.empty((rows, cols), dtype=np.uint16 if out_dtype == BF16 else np.float32)
    sb = sign_bits_from_signs(signs)
    mb = None if maskbits is None else np.ascontiguousarray(maskbits, dtype=np.uint8)
    rc = lib().qo_masked_hadamard_bwd(_ptr(g), dt, rows, cols, hd, scale_dtype, _ptr(sb), _ptr(mb),
                                      _ptr(out), out_dtype)
    if rc != 0:
        raise ValueError(f"qo_masked_hadamard_bwd rc={rc}")
    return out


def rmsnorm(x, gain, eps):
    """(normalised * gain as float32 [rows, cols], per-row factor) of src/models/llama.py:64-75 in the canonical order."""
    x = np.ascontiguousarray(x)
    rows, cols = x.shape
    gain = np.ascontiguousarray(gain, dtype=np.float32)
    out = np.empty((rows, cols), dtype=np.float32)
    factor = np.empty(rows, dtype=np.float32)
    rc = lib().qo_rmsnorm(_ptr(x), _dtype_of(x), _ptr(gain), float(eps), rows, cols, _ptr(out), _ptr(factor))
    assert rc == 0, rc
    return out, factor


def swiglu(h12):
    """silu(up) * gate of a [rows, 2 * hidden] tensor (up first), in h12's dtype (src/models/llama.py:113-114)."""
    h12 = np.ascontiguousarray(h12)
    rows, two = h12.shape
    out = np.empty((rows, two // 2), dtype=h12.dtype)
    rc = lib().qo_swiglu(_ptr(h12), _dtype_of(h12), rows, two // 2, _ptr(out))
    assert rc == 0, rc
    return out


def exp_fixed(z):
    return np.float32(lib().qo_exp(float(np.float32(z))))


def silu(x):
    return np.float32(lib().qo_silu(float(np.float32(x))))


def rtn_code(A):
    return lib().qo_rtn_code(float(A))


def sr_code(A, u):
    return lib().qo_sr_code(float(A), float(u))


def div_four_thirds(g):
    return np.float32(lib().qo_div_four_thirds(float(g)))


# ---------------------------------------------------------------------------------------------
# packed-format helpers (pure numpy)
# ---------------------------------------------------------------------------------------------
def unpack_codes(codes):
    """[R, C/2] bytes -> [R, C] nibbles; element 2i is the low nibble of byte i."""
    lo = codes & 0x0F
    hi = codes >> 4
    return np.stack([lo, hi], axis=-1).reshape(codes.shape[0], -1)


def unpack_mask(maskbits):
    """[R, C/8] bytes -> [R, C] bool; bit i of byte j is element 8j+i
    (notebooks/benchmark_mxfp4.ipynb, _unpack_mask)."""
    bits = (maskbits[..., None] >> np.arange(8, dtype=np.uint8)) & 1
    return bits.reshape(maskbits.shape[0], -1).astype(bool)


def code_values(nibbles):
    v = E2M1_VALUES[nibbles & 7]
    return np.where(nibbles & 8, -v, v).astype(np.float32)


# ---------------------------------------------------------------------------------------------
# independent numpy restatement (matmul form) -- used to pin the C oracle, never by the product
# ---------------------------------------------------------------------------------------------
def sylvester(hd):
    """H[i,j] = (-1)^popcount(i&j), the matrix hadamard_transform(eye) yields (mxfp4.py:42-44)."""
    i = np.arange(hd)
    pc = np.array([[bin(a & b).count("1") for b in i] for a in i])
    return np.where(pc % 2 == 0, 1.0, -1.0)


def np_rotate(xf, hd, c, signs=None):
    """xf float32 [R,C]; dense (x.view(-1,hd) @ S) in float64, rounded once to fp32, then *c, signs."""
    S = sylvester(hd)
    v = (xf.astype(np.float64).reshape(-1, hd) @ S).astype(np.float32)
    v = (v * np.float32(c)).astype(np.float32)
    if signs is not None:
        v = v * np.asarray(signs, dtype=np.float32)[None, :]
    return v.reshape(xf.shape)


_RTN_THRESH = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
_SR_THRESH = np.array([0.5, 1.0, 1.5, 2.0, 3.0, 4.0], dtype=np.float32)


def np_rtn_mag(A):
    """number of thresholds strictly below A (ties toward zero)."""
    return np.searchsorted(_RTN_THRESH, A, side="left").astype(np.uint8)


def np_sr_mag(A, u):
    lo = np.searchsorted(_SR_THRESH, A, side="left")
    vlo = E2M1_VALUES[lo]
    vhi = E2M1_VALUES[lo + 1]
    p = (A - vlo) / (vhi - vlo)
    return (lo + (u < p)).astype(np.uint8)


def np_quantize_rotated(g, mode, u=None):
    """g float32 [R,C] already rotated.  Returns nibbles [R,C], scale bytes [R,C/32], keep [R,C],
    dequant f32 [R,C]."""
    R, C = g.shape
    gg = g.reshape(R, C // 32, 32)
    with np.errstate(all="ignore"):
        if mode in (QUEST_RTN, QUEST_SR):
            sd = np.std(gg.astype(np.float64), axis=-1)  # population std, as ipynb quantize_quest
            s = (QUEST_G * sd.astype(np.float32)).astype(np.float32) + np.float32(1e-8)
            E = np.floor(np.log2(s.astype(np.float64))).astype(np.int32)
            scale = np.ldexp(np.float32(1), E).astype(np.float32)
            t = (gg / scale[..., None]).astype(np.float32)
            byte = (E + 127).astype(np.uint8)
        else:
            a = np.max(np.abs(gg), axis=-1)
            k = np.floor(np.log2(a.astype(np.float64))).astype(np.int64) - 2
            k = np.where(a > 0, k, -127).astype(np.int32)
            scale = (np.ldexp(np.float32(1), k) / np.float32(0.75)).astype(np.float32)
            t = (gg / scale[..., None]).astype(np.float32)
            byte = (k + 127).astype(np.uint8)
            zero = a == 0
            t[zero] = np.nan
    A = np.abs(t)
    if mode in (ABSMAX_SR, QUEST_SR):
        Aq = np.where(np.isnan(A), np.float32(0), A)
        mag = np_sr_mag(np.minimum(Aq, np.float32(1e30)), u.reshape(gg.shape))
        mag = np.where(np.isnan(A), 0, np.minimum(mag, 7)).astype(np.uint8)
    else:
        mag = np.where(np.isnan(A), 0, np_rtn_mag(np.where(np.isnan(A), 0, A))).astype(np.uint8)
    neg = ~(t > 0)
    nib = (mag | (neg.astype(np.uint8) << 3)).astype(np.uint8)
    keep = A < 6
    deq = (code_values(nib) * scale[..., None]).astype(np.float32)
    if mode in (ABSMAX_RTN, ABSMAX_SR):
        deq[a == 0] = -0.0
    return nib.reshape(R, C), byte, keep.reshape(R, C), deq.reshape(R, C)
