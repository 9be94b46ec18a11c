"""Tensor-level wrappers over the C ABI: allocate outputs with torch, pass raw device pointers and
the current HIP stream.  PyTorch is only the allocator and stream provider here."""
import ctypes

import torch

from . import _lib
from ._lib import (QM_ABSMAX_RTN, QM_ABSMAX_SR, QM_BF16, QM_F32, QM_LAYOUT_ROWMAJOR, QM_LAYOUT_TILED,  # noqa: F401
                   QM_QUEST_RTN, QM_QUEST_SR)

FOUR_THIRDS = float(torch.tensor(1.0 / 0.75, dtype=torch.float32))


def _dtype_code(dt):
    if dt == torch.bfloat16:
        return QM_BF16
    if dt == torch.float32:
        return QM_F32
    raise TypeError(f"quartet_amd kernels take bfloat16 or float32 tensors, got {dt}")


def _torch_dtype(code):
    return torch.bfloat16 if code == QM_BF16 else torch.float32


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise _lib.QuartetHipError("quartet_amd kernels need tensors on the GPU (no CPU path exists)")


def sign_words(sign_bits):
    """sign_bits: python int bit mask (bit j = column j negated) or None -> ctypes uint32[4] or None."""
    if sign_bits is None or sign_bits == 0:
        return None
    return (ctypes.c_uint32 * 4)(*[(sign_bits >> (32 * i)) & 0xFFFFFFFF for i in range(4)])


def tile_codes(codes):
    """Row-major code bytes [R, C/2] -> the tiled layout [R/16][C/128][16][64], returned with the same shape."""
    R, B = codes.shape
    return codes.view(R // 16, 16, B // 64, 64).permute(0, 2, 1, 3).contiguous().view(R, B)


def untile_codes(codes):
    """Inverse of tile_codes: tiled code bytes (held as an [R, C/2] tensor) -> row-major [R, C/2]."""
    R, B = codes.shape
    return codes.view(R // 16, B // 64, 16, 64).permute(0, 2, 1, 3).contiguous().view(R, B)


def _layout(tiled):
    return QM_LAYOUT_TILED if tiled else QM_LAYOUT_ROWMAJOR


def quantize_mxfp4(x, hadamard_dim=32, sign_bits=None, mode=QM_QUEST_RTN, transposed_in=False, u=None, seed=0,
                   want_mask=False, want_dequant=False, tiled=False):
    """x: 2-D contiguous tensor.  Returns (codes [R,C/2] u8, scales [R,C/32] u8, maskbits [R,C/8] u8 | None,
    dequant [R,C] like x | None) for the logical [R,C] tensor (x, or x.T when transposed_in).  With `tiled` the
    code bytes come in the tiled layout (see tile_codes); scales and mask stay row-major."""
    _require_cuda(x, u)
    assert x.dim() == 2 and x.is_contiguous()
    rows, cols = (x.shape[1], x.shape[0]) if transposed_in else x.shape
    dev = x.device
    codes = torch.empty((rows, cols // 2), dtype=torch.uint8, device=dev)
    scales = torch.empty((rows, cols // 32), dtype=torch.uint8, device=dev)
    mask = torch.empty((rows, cols // 8), dtype=torch.uint8, device=dev) if want_mask else None
    deq = torch.empty((rows, cols), dtype=x.dtype, device=dev) if want_dequant else None
    if u is not None:
        assert u.dtype == torch.float32 and u.is_contiguous() and u.numel() == rows * cols
    rc = _lib.lib().qm_quantize_mxfp4(_ptr(x), _dtype_code(x.dtype), rows, cols, hadamard_dim, sign_words(sign_bits),
                                      mode, int(transposed_in), _ptr(u), seed, _ptr(codes), _ptr(scales), _ptr(mask),
                                      _ptr(deq), _layout(tiled), _stream())
    _lib.check(rc, "qm_quantize_mxfp4")
    return codes, scales, mask, deq


def _matrix_arg(matrix, device):
    """A dense rotation as the kernels read it: contiguous fp32 [32, 32] on the tensors' device."""
    m = matrix.detach().to(device=device, dtype=torch.float32).contiguous()
    if tuple(m.shape) != (32, 32):
        raise _lib.QuartetHipError(f"a dense rotation must be 32 x 32, got {tuple(m.shape)}")
    return m


def quantize_mxfp4_dense(x, matrix, mode=QM_ABSMAX_RTN, transposed_in=False, seed=0, want_mask=False, want_dequant=False,
                         tiled=False):
    """quantize_mxfp4 with a dense 32 x 32 rotation (`matrix`, H[k][j]) applied to every group of 32 in place of the
    Hadamard block.  Same return value."""
    _require_cuda(x)
    assert x.dim() == 2 and x.is_contiguous()
    rows, cols = (x.shape[1], x.shape[0]) if transposed_in else x.shape
    dev = x.device
    m = _matrix_arg(matrix, dev)
    codes = torch.empty((rows, cols // 2), dtype=torch.uint8, device=dev)
    scales = torch.empty((rows, cols // 32), dtype=torch.uint8, device=dev)
    mask = torch.empty((rows, cols // 8), dtype=torch.uint8, device=dev) if want_mask else None
    deq = torch.empty((rows, cols), dtype=x.dtype, device=dev) if want_dequant else None
    rc = _lib.lib().qm_quantize_mxfp4_dense(_ptr(x), _dtype_code(x.dtype), rows, cols, _ptr(m), mode, int(transposed_in), seed,
                                            _ptr(codes), _ptr(scales), _ptr(mask), _ptr(deq), _layout(tiled), _stream())
    _lib.check(rc, "qm_quantize_mxfp4_dense")
    return codes, scales, mask, deq


def requantize_transposed_mxfp4_dense(codes, scales, matrix, post=1.0, val_dtype=torch.bfloat16, mode=QM_ABSMAX_SR, seed=0,
                                      want_dequant=False, tiled_in=False, tiled_out=False):
    """requantize_transposed_mxfp4 with a dense 32 x 32 rotation.  Same return value."""
    _require_cuda(codes, scales)
    assert codes.is_contiguous() and scales.is_contiguous()
    R, C = codes.shape[0], codes.shape[1] * 2
    dev = codes.device
    m = _matrix_arg(matrix, dev)
    codes_out = torch.empty((C, R // 2), dtype=torch.uint8, device=dev)
    scales_out = torch.empty((C, R // 32), dtype=torch.uint8, device=dev)
    deq = torch.empty((C, R), dtype=val_dtype, device=dev) if want_dequant else None
    rc = _lib.lib().qm_requantize_transposed_mxfp4_dense(_ptr(codes), _ptr(scales), R, C, post, _dtype_code(val_dtype), _ptr(m), mode,
                                                         seed, _ptr(codes_out), _ptr(scales_out), _ptr(deq), _layout(tiled_in),
                                                         _layout(tiled_out), _stream())
    _lib.check(rc, "qm_requantize_transposed_mxfp4_dense")
    return codes_out, scales_out, deq


def requantize_transposed_mxfp4(codes, scales, post=1.0, val_dtype=torch.bfloat16, hadamard_dim=32, sign_bits=None,
                                mode=QM_ABSMAX_SR, u=None, seed=0, want_dequant=False, tiled_in=False, tiled_out=False):
    """codes [R,C/2], scales [R,C/32] -> (codes [C,R/2], scales [C,R/32], dequant [C,R] | None)."""
    _require_cuda(codes, scales, u)
    assert codes.is_contiguous() and scales.is_contiguous()
    R, C = codes.shape[0], codes.shape[1] * 2
    dev = codes.device
    codes_out = torch.empty((C, R // 2), dtype=torch.uint8, device=dev)
    scales_out = torch.empty((C, R // 32), dtype=torch.uint8, device=dev)
    deq = torch.empty((C, R), dtype=val_dtype, device=dev) if want_dequant else None
    rc = _lib.lib().qm_requantize_transposed_mxfp4(_ptr(codes), _ptr(scales), R, C, post, _dtype_code(val_dtype),
                                                   hadamard_dim, sign_words(sign_bits), mode, _ptr(u), seed,
                                                   _ptr(codes_out), _ptr(scales_out), _ptr(deq), _layout(tiled_in),
                                                   _layout(tiled_out), _stream())
    _lib.check(rc, "qm_requantize_transposed_mxfp4")
    return codes_out, scales_out, deq


def gemm_mxfp4_tn(a_codes, a_scales, b_codes, b_scales, alpha=1.0, out_dtype=torch.bfloat16, a_tiled=False, b_tiled=False,
                  split_k=True):
    """[M,K/2],[M,K/32] x [N,K/2],[N,K/32] -> alpha * A @ B^T as [M,N] of out_dtype.  With `split_k` the library
    may cut a long-K, few-tile product into K ranges (scratch is allocated here when it asks for it)."""
    _require_cuda(a_codes, a_scales, b_codes, b_scales)
    M, K = a_codes.shape[0], a_codes.shape[1] * 2
    N = b_codes.shape[0]
    if b_codes.shape[1] * 2 != K:
        raise _lib.QuartetHipError(f"gemm_mxfp4_tn: contraction sizes differ ({K} vs {b_codes.shape[1] * 2})")
    c = torch.empty((M, N), dtype=out_dtype, device=a_codes.device)
    ws_bytes = _lib.lib().qm_gemm_workspace_bytes(M, N, K) if split_k else 0
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=a_codes.device) if ws_bytes else None
    rc = _lib.lib().qm_gemm_mxfp4_tn(_ptr(a_codes), _ptr(a_scales), _ptr(b_codes), _ptr(b_scales), M, N, K, alpha,
                                     _ptr(c), _dtype_code(out_dtype), _layout(a_tiled), _layout(b_tiled), _ptr(ws), ws_bytes,
                                     _stream())
    _lib.check(rc, "qm_gemm_mxfp4_tn")
    return c


def gemm_fuses_rotation(a_scales, b_scales, M, N, K):
    """Whether gemm_mxfp4_tn_rotated serves this product (the persistent kernel, no cut into K ranges)."""
    return bool(_lib.lib().qm_gemm_fuses_rotation(_ptr(a_scales), _ptr(b_scales), M, N, K))


def gemm_mxfp4_tn_rotated(a_codes, a_scales, b_codes, b_scales, maskbits, alpha=1.0, scale_dtype=torch.bfloat16, sign_bits=None,
                          a_tiled=False, b_tiled=False):
    """masked_hadamard_bwd(gemm_mxfp4_tn(..., bf16), 32, scale_dtype, sign_bits, maskbits) in one launch: the product's
    epilogue rounds the tile to bf16, masks it and rotates it on the matrix pipe.  [M,N] bf16.  Raises for shapes the
    fused kernel does not serve (gemm_fuses_rotation tells)."""
    _require_cuda(a_codes, a_scales, b_codes, b_scales, maskbits)
    M, K = a_codes.shape[0], a_codes.shape[1] * 2
    N = b_codes.shape[0]
    if b_codes.shape[1] * 2 != K:
        raise _lib.QuartetHipError(f"gemm_mxfp4_tn_rotated: contraction sizes differ ({K} vs {b_codes.shape[1] * 2})")
    assert maskbits.shape == (M, N // 8) and maskbits.is_contiguous()
    c = torch.empty((M, N), dtype=torch.bfloat16, device=a_codes.device)
    rc = _lib.lib().qm_gemm_mxfp4_tn_rotated(_ptr(a_codes), _ptr(a_scales), _ptr(b_codes), _ptr(b_scales), M, N, K, alpha, _ptr(c),
                                             _layout(a_tiled), _layout(b_tiled), _ptr(maskbits), sign_words(sign_bits),
                                             _dtype_code(scale_dtype), _stream())
    _lib.check(rc, "qm_gemm_mxfp4_tn_rotated")
    return c


def gemm_mxfp4_bf16_nn_supported(M, N, K):
    return K > 0 and K % 64 == 0 and N % 8 == 0 and M > 0 and N > 0


def gemm_mxfp4_bf16_nn(a_codes, a_scales, b, alpha=1.0, out_dtype=torch.bfloat16):
    """[M,K/2],[M,K/32] packed MXFP4 (row-major) x b [K,N] bf16 row-major -> alpha * A @ b as [M,N] of out_dtype."""
    _require_cuda(a_codes, a_scales, b)
    M, K = a_codes.shape[0], a_codes.shape[1] * 2
    if b.dtype != torch.bfloat16 or b.dim() != 2 or b.shape[0] != K or not b.is_contiguous():
        raise _lib.QuartetHipError(f"gemm_mxfp4_bf16_nn: b must be a contiguous bf16 [{K}, N] tensor, got {tuple(b.shape)} {b.dtype}")
    N = b.shape[1]
    c = torch.empty((M, N), dtype=out_dtype, device=a_codes.device)
    rc = _lib.lib().qm_gemm_mxfp4_bf16_nn(_ptr(a_codes), _ptr(a_scales), _ptr(b), M, N, K, alpha, _ptr(c), _dtype_code(out_dtype),
                                          _stream())
    _lib.check(rc, "qm_gemm_mxfp4_bf16_nn")
    return c


_noalloc_prepared = set()


def gemm_noalloc_prepare():
    """Look up the current device's copy of the library's built-in scratch array (once per device; the one step of the
    allocation-free product that may make the HIP runtime place the library's device image in GPU memory).  Must not
    run under stream capture."""
    dev = torch.cuda.current_device()
    if dev not in _noalloc_prepared:
        _lib.check(_lib.lib().qm_gemm_noalloc_prepare(), "qm_gemm_noalloc_prepare")
        _noalloc_prepared.add(dev)


def gemm_mxfp4_tn_noalloc(a_codes, a_scales, b_codes, b_scales, alpha, out):
    """The same product through the library's allocation-free entry point: `out` [M,N] (bf16 or fp32) is written in
    place and split-K partial sums go to the library's built-in device scratch.  Row-major code bytes."""
    _require_cuda(a_codes, a_scales, b_codes, b_scales, out)
    M, K = a_codes.shape[0], a_codes.shape[1] * 2
    N = b_codes.shape[0]
    assert out.shape == (M, N) and out.is_contiguous() and b_codes.shape[1] * 2 == K
    with torch.cuda.device(out.device):
        gemm_noalloc_prepare()
    rc = _lib.lib().qm_gemm_mxfp4_tn_noalloc(_ptr(a_codes), _ptr(a_scales), _ptr(b_codes), _ptr(b_scales), M, N, K, alpha,
                                             _ptr(out), _dtype_code(out.dtype), QM_LAYOUT_ROWMAJOR, QM_LAYOUT_ROWMAJOR,
                                             _stream())
    _lib.check(rc, "qm_gemm_mxfp4_tn_noalloc")
    return out


PHASE_STAMPS = 32   # QM_DIAG_PHASE_STAMPS


def gemm_tile_phases(a_codes, a_scales, b_codes, b_scales, alpha=1.0, a_tiled=False, b_tiled=False, maskbits=None):
    """Measurement aid: one launch of the persistent tile kernel's stamping instantiation.  Returns (c [M,N] bf16,
    stamps int64 [workgroups, 32] on the host): per workgroup the shader clock at entry, at the start of its tile loop,
    then after the K loop and after the epilogue of each of its tiles (unused slots are zero).  With `maskbits` [M, N/8]
    the instantiation whose epilogue carries the masked inverse rotation (c is then the rotated product)."""
    _require_cuda(a_codes, a_scales, b_codes, b_scales, maskbits)
    M, K = a_codes.shape[0], a_codes.shape[1] * 2
    N = b_codes.shape[0]
    assert b_codes.shape[1] * 2 == K
    c = torch.empty((M, N), dtype=torch.bfloat16, device=a_codes.device)
    stamps = torch.zeros((1024, PHASE_STAMPS), dtype=torch.int64, device=a_codes.device)
    groups = _lib.lib().qm_diag_gemm_tile_phases(_ptr(a_codes), _ptr(a_scales), _ptr(b_codes), _ptr(b_scales), M, N, K, alpha,
                                                 _ptr(c), _layout(a_tiled), _layout(b_tiled), _ptr(maskbits), _ptr(stamps),
                                                 stamps.numel() * 8, _stream())
    if groups < 0:
        _lib.check(int(groups), "qm_diag_gemm_tile_phases")
    torch.cuda.synchronize()
    return c, stamps[:groups].cpu()


def mfma_only(operand_bytes, iters):
    """Measurement aid: `iters` iterations of the FP4 matrix instruction alone on every CU, fed with bytes of
    `operand_bytes` (uint8, at least 32 KiB per CU).  Returns the number of 32 x 32 x 64 instructions issued."""
    _require_cuda(operand_bytes)
    assert operand_bytes.dtype == torch.uint8 and operand_bytes.is_contiguous()
    sink = torch.empty(1 << 18, dtype=torch.float32, device=operand_bytes.device)
    n = _lib.lib().qm_diag_mfma_only(_ptr(operand_bytes), operand_bytes.numel(), _ptr(sink), sink.numel() * 4, iters, _stream())
    if n < 0:
        _lib.check(int(n), "qm_diag_mfma_only")
    return n


def masked_hadamard_bwd(g, hadamard_dim=32, scale_dtype=torch.bfloat16, sign_bits=None, maskbits=None, out_dtype=None,
                        out=None):
    """g [R,C] -> ((g*mask).view(-1,hd) @ H^T) as [R,C] of out_dtype (default g.dtype); `out` may be pre-allocated."""
    _require_cuda(g, maskbits)
    assert g.dim() == 2 and g.is_contiguous()
    out_dtype = g.dtype if out_dtype is None else out_dtype
    if out is None:
        out = torch.empty(g.shape, dtype=out_dtype, device=g.device)
    assert out.shape == g.shape and out.dtype == out_dtype and out.is_contiguous()
    rc = _lib.lib().qm_masked_hadamard_bwd(_ptr(g), _dtype_code(g.dtype), g.shape[0], g.shape[1], hadamard_dim,
                                           _dtype_code(scale_dtype), sign_words(sign_bits), _ptr(maskbits), _ptr(out),
                                           _dtype_code(out_dtype), _stream())
    _lib.check(rc, "qm_masked_hadamard_bwd")
    return out


def dequantize_mxfp4(codes, scales, post=1.0, out_dtype=torch.float32):
    _require_cuda(codes, scales)
    R, C = codes.shape[0], codes.shape[1] * 2
    out = torch.empty((R, C), dtype=out_dtype, device=codes.device)
    rc = _lib.lib().qm_dequantize_mxfp4(_ptr(codes), _ptr(scales), R, C, post, _ptr(out), _dtype_code(out_dtype),
                                        _stream())
    _lib.check(rc, "qm_dequantize_mxfp4")
    return out


def packed_operand_buffer(rows, cols, device):
    """Uninitialised byte buffer for one packed operand (codes, scales, mask bits of a [rows, cols] tensor)."""
    return torch.empty(_lib.lib().qm_packed_operand_bytes(rows, cols), dtype=torch.uint8, device=device)


QM_W_IS_PACKED, QM_X_IS_PACKED = 1, 2


def quantize_dense_into_packed(x2, matrix, tiled):
    """Quest RTN + clip mask of x2 [rows, cols] under a dense 32 x 32 rotation, written into a fresh packed-operand buffer
    (what linear_forward fills for a Hadamard rotation): the forward quantizer of a layer whose quantizer holds the matrix
    of rerotate="O32"."""
    _require_cuda(x2)
    assert x2.dim() == 2 and x2.is_contiguous()
    rows, cols = x2.shape
    packed = packed_operand_buffer(rows, cols, x2.device)
    off = (ctypes.c_size_t * 3)()
    _lib.check(_lib.lib().qm_packed_operand_offsets(rows, cols, off), "qm_packed_operand_offsets")
    m = _matrix_arg(matrix, x2.device)
    base = packed.data_ptr()
    rc = _lib.lib().qm_quantize_mxfp4_dense(_ptr(x2), _dtype_code(x2.dtype), rows, cols, _ptr(m), QM_QUEST_RTN, 0, 0, base + off[0],
                                            base + off[1], base + off[2], None, _layout(tiled), _stream())
    _lib.check(rc, "qm_quantize_mxfp4_dense")
    return packed


def linear_forward(x2, w2, hd_x, signs_x, hd_w, signs_w, out_dtype, tiled, packed_w=None, packed_x=None, rows=None):
    """Whole forward pass of a Quartet linear in one foreign call: quantize x [T,I] and w [O,I] (quest RTN + clip
    mask), y = Q(x) Q(w)^T.  Returns (y [T,O], packed_x, packed_w): the byte buffers the backward pass reads.  A
    `packed_w` that an earlier call with the same weight, signs and layout returned is reused instead of quantizing
    the weight again; a `packed_x` written by a fused producer (rmsnorm_quantize, swiglu_quantize) of a [rows, I]
    tensor replaces x2 (pass None)."""
    _require_cuda(x2, w2, packed_w, packed_x)
    assert w2.is_contiguous()
    O, I = w2.shape
    if packed_x is None:
        assert x2.is_contiguous() and x2.shape[1] == I
        T = x2.shape[0]
    else:
        assert x2 is None and rows is not None
        T = rows
    L = _lib.lib()
    flags = (QM_W_IS_PACKED if packed_w is not None else 0) | (QM_X_IS_PACKED if packed_x is not None else 0)
    if packed_x is None:
        packed_x = packed_operand_buffer(T, I, w2.device)
    if packed_w is None:
        packed_w = packed_operand_buffer(O, I, w2.device)
    y = torch.empty((T, O), dtype=out_dtype, device=w2.device)
    rc = L.qm_linear_forward(_ptr(x2), _dtype_code(x2.dtype) if x2 is not None else 0, _ptr(w2), _dtype_code(w2.dtype), T, I, O, hd_x,
                             sign_words(signs_x), hd_w, sign_words(signs_w), _ptr(packed_x), packed_x.numel(), _ptr(packed_w),
                             packed_w.numel(), flags, _ptr(y), _dtype_code(out_dtype), _layout(tiled), _stream())
    _lib.check(rc, "qm_linear_forward")
    return y, packed_x, packed_w


def rmsnorm_quantize(x2, gain, eps, signs, tiled, add=None):
    """Q(rmsnorm(x2) * gain) without writing the normalised tensor: (packed operand buffer, per-row factor fp32).  With
    `add` (x2 fp32, add like x2 in bf16 or fp32) the norm's input is x2 + add, returned as a third value."""
    _require_cuda(x2, gain, add)
    assert x2.is_contiguous() and gain.is_contiguous() and gain.dtype == torch.float32 and gain.shape == (x2.shape[1],)
    rows, cols = x2.shape
    packed = packed_operand_buffer(rows, cols, x2.device)
    factor = torch.empty(rows, dtype=torch.float32, device=x2.device)
    x_sum = None
    if add is not None:
        assert add.is_contiguous() and add.shape == x2.shape and x2.dtype == torch.float32
        x_sum = torch.empty_like(x2)
    rc = _lib.lib().qm_rmsnorm_quantize_mxfp4(_ptr(x2), _dtype_code(x2.dtype), _ptr(add), _dtype_code(add.dtype) if add is not None else 0,
                                              _ptr(x_sum), _ptr(gain), float(eps), rows, cols, sign_words(signs), _ptr(packed),
                                              packed.numel(), _ptr(factor), _layout(tiled), _stream())
    _lib.check(rc, "qm_rmsnorm_quantize_mxfp4")
    return (packed, factor) if add is None else (packed, factor, x_sum)


def swiglu_quantize(h12, signs, tiled):
    """Q(silu(up) * gate) of h12 [rows, 2 hidden] = (up, gate) without writing the product: packed operand buffer."""
    _require_cuda(h12)
    assert h12.is_contiguous() and h12.shape[1] % 2 == 0
    rows, hidden = h12.shape[0], h12.shape[1] // 2
    packed = packed_operand_buffer(rows, hidden, h12.device)
    rc = _lib.lib().qm_swiglu_quantize_mxfp4(_ptr(h12), _dtype_code(h12.dtype), rows, hidden, sign_words(signs), _ptr(packed),
                                             packed.numel(), _layout(tiled), _stream())
    _lib.check(rc, "qm_swiglu_quantize_mxfp4")
    return packed


def packed_mask_bits(packed, rows, cols):
    """The clip-mask bits [rows, cols/8] inside a packed operand buffer (a view)."""
    off = (ctypes.c_size_t * 3)()
    _lib.check(_lib.lib().qm_packed_operand_offsets(rows, cols, off), "qm_packed_operand_offsets")
    return packed[off[2]: off[2] + rows * cols // 8].view(rows, cols // 8)


def rmsnorm_backward(gy, x2, gain, factor, maskbits=None, signs=0, scale_dtype=torch.float32, skip=None, want_bf16_copy=False):
    """gy [rows, cols] (gradient of the normalised, scaled tensor) -> (dx like x2, dgain fp32 [cols]).  With `maskbits`
    (and the rotation's `signs`, `scale_dtype`), gy is the gradient in the activation quantizer's rotated basis and its
    straight-through backward is applied first, inside the kernel.  `skip` (like x2) is added to dx: the gradient of a
    residual connection around the norm.  `want_bf16_copy`: returns dx rounded to bf16 as a third value."""
    _require_cuda(gy, x2, gain, factor, maskbits, skip)
    assert skip is None or (skip.is_contiguous() and skip.shape == x2.shape and skip.dtype == x2.dtype)
    assert gy.is_contiguous() and x2.is_contiguous() and gy.shape == x2.shape
    rows, cols = x2.shape
    L = _lib.lib()
    nbytes = L.qm_rmsnorm_backward_workspace_bytes(rows, cols)
    work = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=x2.device)
    dx = torch.empty_like(x2)
    dgain = torch.empty(cols, dtype=torch.float32, device=x2.device)
    dx_bf16 = torch.empty(x2.shape, dtype=torch.bfloat16, device=x2.device) if want_bf16_copy else None
    rc = L.qm_rmsnorm_backward(_ptr(gy), _dtype_code(gy.dtype), _ptr(x2), _dtype_code(x2.dtype), _ptr(gain), _ptr(factor), rows, cols,
                               _ptr(maskbits), sign_words(signs), _dtype_code(scale_dtype), _ptr(skip), _ptr(dx), _ptr(dx_bf16),
                               _ptr(dgain), _ptr(work), nbytes, _stream())
    _lib.check(rc, "qm_rmsnorm_backward")
    return (dx, dgain, dx_bf16) if want_bf16_copy else (dx, dgain)


def swiglu_backward(g, h12, maskbits=None, signs=0, scale_dtype=torch.float32):
    """g [rows, hidden] (gradient of silu(up) * gate) -> gradient of h12 [rows, 2 hidden], in h12's dtype; `maskbits`
    as for rmsnorm_backward."""
    _require_cuda(g, h12, maskbits)
    assert g.is_contiguous() and h12.is_contiguous() and h12.shape == (g.shape[0], 2 * g.shape[1])
    d = torch.empty_like(h12)
    rc = _lib.lib().qm_swiglu_backward(_ptr(g), _dtype_code(g.dtype), _ptr(h12), _dtype_code(h12.dtype), g.shape[0], g.shape[1],
                                       _ptr(maskbits), sign_words(signs), _dtype_code(scale_dtype), _ptr(d), _stream())
    _lib.check(rc, "qm_swiglu_backward")
    return d


def rope_split_qkv(qkv2, table, n_embd, head_dim, seq_len, out_dtype):
    """qkv2 [rows, 3 n_embd] -> (q, k, v) [rows, n_embd] of out_dtype, q and k rotated pairwise by table [seq_len, head_dim/2, 2]."""
    _require_cuda(qkv2, table)
    assert qkv2.is_contiguous() and table.is_contiguous() and table.dtype == torch.float32
    assert qkv2.shape[1] == 3 * n_embd and tuple(table.shape) == (seq_len, head_dim // 2, 2)
    rows = qkv2.shape[0]
    q, k, v = (torch.empty((rows, n_embd), dtype=out_dtype, device=qkv2.device) for _ in range(3))
    rc = _lib.lib().qm_rope_split_qkv(_ptr(qkv2), _dtype_code(qkv2.dtype), rows, seq_len, n_embd, head_dim, _ptr(table), _ptr(q),
                                      _ptr(k), _ptr(v), _dtype_code(out_dtype), _stream())
    _lib.check(rc, "qm_rope_split_qkv")
    return q, k, v


def rope_merge_qkv_grad(dq, dk, dv, table, n_embd, head_dim, seq_len, out_dtype):
    """Gradients of rope_split_qkv's outputs, each [rows, n_embd] -> gradient of its input [rows, 3 n_embd] of out_dtype."""
    _require_cuda(dq, dk, dv, table)
    assert dq.is_contiguous() and dk.is_contiguous() and dv.is_contiguous() and dq.dtype == dk.dtype == dv.dtype
    rows = dq.shape[0]
    d_qkv = torch.empty((rows, 3 * n_embd), dtype=out_dtype, device=dq.device)
    rc = _lib.lib().qm_rope_merge_qkv_grad(_ptr(dq), _ptr(dk), _ptr(dv), _dtype_code(dq.dtype), rows, seq_len, n_embd, head_dim,
                                           _ptr(table), _ptr(d_qkv), _dtype_code(out_dtype), _stream())
    _lib.check(rc, "qm_rope_merge_qkv_grad")
    return d_qkv


def linear_backward(e2, packed_x, packed_w, T, I, O, hd_x, signs_x, hd_w, signs_w, hd_g, signs_g, mode, seeds, x_val_dtype,
                    w_val_dtype, mid_dtype, x_scale_dtype, w_scale_dtype, tiled, gx_rotated=False, gw_dtype=None, g_matrix=None,
                    seed_base=None, gw_rotated=False):
    """Whole backward pass in one foreign call: e [T,O] -> (gx [T,I], gw [O,I]) of mid_dtype.  With `gx_rotated`, gx is
    still in the rotated basis of the activation quantizer: its masked inverse rotation is left to the kernel that
    consumes gx (rmsnorm_backward / swiglu_backward with `maskbits`); with `gw_rotated` likewise gw (mid_dtype) in the
    weight quantizer's rotated basis.  `gw_dtype` = float32 with a bf16 mid_dtype returns
    gw as the bf16-rounded values widened to fp32 (the cast autograd would apply for an fp32 weight) in the same pass.
    `seed_base`: a one-element int64 tensor on the GPU whose value the gradient quantizers add to their seeds when they
    run (a step replayed from a captured graph draws fresh random streams if the graph also increments it)."""
    _require_cuda(e2, packed_x, packed_w, seed_base)
    if seed_base is not None:
        assert seed_base.dtype == torch.int64 and seed_base.numel() >= 1 and seed_base.is_contiguous()
    assert e2.is_contiguous() and e2.shape == (T, O)
    L = _lib.lib()
    mid = _dtype_code(mid_dtype)
    nbytes = L.qm_linear_backward_workspace_bytes(T, I, O, mid)
    work = torch.empty(nbytes, dtype=torch.uint8, device=e2.device)
    gx = torch.empty((T, I), dtype=mid_dtype, device=e2.device)
    gw_dtype = mid_dtype if gw_dtype is None or mid_dtype != torch.bfloat16 or gw_rotated else gw_dtype
    gw = torch.empty((O, I), dtype=gw_dtype, device=e2.device)
    rc = L.qm_linear_backward_seeded(_ptr(e2), _dtype_code(e2.dtype), T, I, O, _ptr(packed_x), _ptr(packed_w), hd_x,
                                     sign_words(signs_x), hd_w, sign_words(signs_w), hd_g, sign_words(signs_g), mode,
                                     (ctypes.c_uint64 * 4)(*seeds), _dtype_code(x_val_dtype), _dtype_code(w_val_dtype), mid,
                                     _dtype_code(x_scale_dtype), _dtype_code(w_scale_dtype), _ptr(work), nbytes, _ptr(gx), _ptr(gw),
                                     _dtype_code(gw_dtype), _layout(tiled), int(bool(gx_rotated)) | (int(bool(gw_rotated)) << 1), _ptr(g_matrix),
                                     _ptr(seed_base), _stream())
    _lib.check(rc, "qm_linear_backward")
    return gx, gw
