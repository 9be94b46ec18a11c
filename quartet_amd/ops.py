"""``torch.library`` operators in the ``quartet::`` namespace over the C ABI.

The reference registers its real-FP4 kernels this way (notebooks/benchmark_mxfp4.ipynb, the cell that defines
``matmul_mxf4_bf16_tn_op``, ``fusedQuantizeMx_op``, ``backward_t_bf16_op`` and ``backward_qt_bf16_op`` with
``torch.library.custom_op`` + ``register_fake``) so that ``torch.compile(fullgraph=True)`` and compiled autograd
can trace through its ``CudaGemm`` Function.  The operators here keep those names, argument orders and result
shapes, with three differences that the packed format of this library dictates:

  * E8M0 scales come back as plain row-major ``[rows, cols/32]`` bytes: no padding to 128x4 and no blocked
    re-ordering (``to_blocked`` has nothing to do), and the GEMM operator takes them in that form;
  * ``fusedQuantizeMx_op`` returns an empty tensor in place of the mask when ``return_mask`` is false (an operator
    result cannot be ``None``);
  * the value an (E2M1 code, E8M0 byte) pair stands for is ``code * 2^(byte-127)`` for the quest quantizer and
    ``code * 2^(byte-127) * 4/3`` for the absmax quantizers, so a product of two absmax operands needs
    ``alpha = 16/9`` (``ALPHA_BWD``), of one absmax and one quest operand ``4/3``.

Two operators that the notebook composes from torch calls are added because the hot path has kernels for them:
``fusedQuantizeMxAbsMax_op`` (row-major absmax quantizer of the gradient) and ``maskedHadamardBwd_op`` (the
straight-through estimator of the forward quantizer).  ``PackedLinearFn`` chains the operators in the order of the
notebook's ``CudaGemm``.

The rotation argument is the dense ``[hd, hd]`` matrix the reference passes around; it must be a Sylvester Hadamard
matrix scaled by ``hd^-1/2`` with negated columns, which is what every quantizer module holds.  Reading its signs
(and the value of an ``alpha`` tensor) takes one device-to-host copy, remembered for as long as that tensor object lives unmodified.
"""
import torch

from . import kernels as K
from .quantizers.mxfp4 import _fresh_seed, register_host_value, remember_host_value, sylvester_sign_bits

ALPHA_FWD = 1.0
ALPHA_BWD = K.FOUR_THIRDS * K.FOUR_THIRDS

def rotation_sign_bits(hadamard_matrix):
    """Bit mask of the negated columns of ``hd^-1/2 * Sylvester * diag(+-1)``; raises for any other matrix."""
    if hadamard_matrix.dim() != 2 or hadamard_matrix.shape[0] != hadamard_matrix.shape[1]:
        raise ValueError(f"rotation must be a square matrix, got shape {tuple(hadamard_matrix.shape)}")
    if hadamard_matrix.shape[0] not in (32, 64, 128):
        raise ValueError(f"rotation size must be 32, 64 or 128, got {hadamard_matrix.shape[0]}")
    bits = sylvester_sign_bits(hadamard_matrix)
    if bits is None:
        raise ValueError("rotation is not a scaled Sylvester Hadamard matrix with negated columns; the packed operators "
                         "do not take dense rotations")
    return bits


def _host_scalar(t):
    return remember_host_value("scalar", t, lambda: float(t.detach().reshape(-1)[0].item()))


_constants = {}


def constant_alpha(value, device):
    """A one-element tensor holding `value` on `device`, created once and remembered together with its host value: the
    operators that take an ``alpha`` tensor then need no device-to-host copy (a copy would synchronise the stream on
    every call and is not allowed while a HIP graph is being captured)."""
    if torch.compiler.is_compiling():   # under tracing the tensor is a graph constant; the operator reads it at run time
        return torch.full((1,), float(value), device=device)
    key = (float(value), torch.device(device))
    t = _constants.get(key)
    if t is None:
        t = torch.full((1,), float(value), device=device)
        _constants[key] = t
    register_host_value("scalar", t, float(value))
    return t


def _rows(x):
    if x.dim() != 2:
        raise ValueError(f"expected a 2-D tensor, got shape {tuple(x.shape)}")
    return x.contiguous()


@torch.library.custom_op("quartet::fusedQuantizeMx_op", mutates_args=(), device_types="cuda")
def fusedQuantizeMx_op(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor,
                       return_mask: bool) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Rotate groups of hd columns, quantize with the quest scale and round-to-nearest.
    [M,K] -> (E2M1 [M,K/2], E8M0 [M,K/32], clip-mask bits [M,K/8] or an empty tensor)."""
    x2 = _rows(x_flat)
    codes, scales, mask, _ = K.quantize_mxfp4(x2, hadamard_matrix.shape[0], rotation_sign_bits(hadamard_matrix),
                                              K.QM_QUEST_RTN, want_mask=return_mask)
    return codes, scales, mask if return_mask else x2.new_empty((0,), dtype=torch.uint8)


@fusedQuantizeMx_op.register_fake
def _(x_flat, hadamard_matrix, return_mask):
    M, Kd = x_flat.shape
    u8 = dict(dtype=torch.uint8, device=x_flat.device)
    return (torch.empty((M, Kd // 2), **u8), torch.empty((M, Kd // 32), **u8),
            torch.empty((M, Kd // 8) if return_mask else (0,), **u8))


@torch.library.custom_op("quartet::fusedQuantizeMxAbsMax_op", mutates_args=(), device_types="cuda")
def fusedQuantizeMxAbsMax_op(x_flat: torch.Tensor, hadamard_matrix: torch.Tensor,
                             stochastic: bool) -> tuple[torch.Tensor, torch.Tensor]:
    """Rotate, scale each group of 32 by its absolute maximum and round (stochastically when asked).
    [M,K] -> (E2M1 [M,K/2], E8M0 [M,K/32])."""
    x2 = _rows(x_flat)
    codes, scales, _, _ = K.quantize_mxfp4(x2, hadamard_matrix.shape[0], rotation_sign_bits(hadamard_matrix),
                                           K.QM_ABSMAX_SR if stochastic else K.QM_ABSMAX_RTN,
                                           seed=_fresh_seed() if stochastic else 0)
    return codes, scales


@fusedQuantizeMxAbsMax_op.register_fake
def _(x_flat, hadamard_matrix, stochastic):
    M, Kd = x_flat.shape
    u8 = dict(dtype=torch.uint8, device=x_flat.device)
    return torch.empty((M, Kd // 2), **u8), torch.empty((M, Kd // 32), **u8)


@torch.library.custom_op("quartet::backward_t_bf16_op", mutates_args=(), device_types="cuda")
def backward_t_bf16_op(grad_output_flat: torch.Tensor, hadamard_matrix: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Quantize the transpose: rotate groups along the row axis of g, absmax scale, stochastic rounding.
    g [M,K] -> (E2M1 [K,M/2], E8M0 [K,M/32])."""
    g2 = _rows(grad_output_flat)
    codes, scales, _, _ = K.quantize_mxfp4(g2, hadamard_matrix.shape[0], rotation_sign_bits(hadamard_matrix),
                                           K.QM_ABSMAX_SR, transposed_in=True, seed=_fresh_seed())
    return codes, scales


@backward_t_bf16_op.register_fake
def _(grad_output_flat, hadamard_matrix):
    M, Kd = grad_output_flat.shape
    u8 = dict(dtype=torch.uint8, device=grad_output_flat.device)
    return torch.empty((Kd, M // 2), **u8), torch.empty((Kd, M // 32), **u8)


@torch.library.custom_op("quartet::backward_qt_bf16_op", mutates_args=(), device_types="cuda")
def backward_qt_bf16_op(x_e2m1: torch.Tensor, x_e8m0: torch.Tensor, h: torch.Tensor,
                        alpha: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """De-quantize to bf16 values times alpha, transpose, rotate along the new row, absmax scale, stochastic rounding.
    (E2M1 [M,K/2], E8M0 [M,K/32]) -> (E2M1 [K,M/2], E8M0 [K,M/32])."""
    if x_e2m1.dim() != 2:
        raise ValueError(f"expected 2-D codes, got shape {tuple(x_e2m1.shape)}")
    codes, scales, _ = K.requantize_transposed_mxfp4(x_e2m1.contiguous(), x_e8m0.contiguous(), _host_scalar(alpha),
                                                     torch.bfloat16, h.shape[0], rotation_sign_bits(h), K.QM_ABSMAX_SR,
                                                     seed=_fresh_seed())
    return codes, scales


@backward_qt_bf16_op.register_fake
def _(x_e2m1, x_e8m0, h, alpha):
    M, half = x_e2m1.shape
    u8 = dict(dtype=torch.uint8, device=x_e2m1.device)
    return torch.empty((half * 2, M // 2), **u8), torch.empty((half * 2, M // 32), **u8)


@torch.library.custom_op("quartet::matmul_mxf4_bf16_tn_op", mutates_args=(), device_types="cuda")
def matmul_mxf4_bf16_tn_op(x: torch.Tensor, w: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor,
                           alpha: torch.Tensor) -> torch.Tensor:
    """alpha * X W^T on the block-scaled FP4 matrix cores.
    (E2M1 [M,K/2], E2M1 [N,K/2], E8M0 [M,K/32], E8M0 [N,K/32]) -> bf16 [M,N]."""
    return K.gemm_mxfp4_tn(x.view(torch.uint8).contiguous(), xs.view(torch.uint8).contiguous(),
                           w.view(torch.uint8).contiguous(), ws.view(torch.uint8).contiguous(), _host_scalar(alpha),
                           torch.bfloat16)


@matmul_mxf4_bf16_tn_op.register_fake
def _(x, w, xs, ws, alpha):
    return x.new_empty((x.shape[0], w.shape[0]), dtype=torch.bfloat16)


@torch.library.custom_op("quartet::maskedHadamardBwd_op", mutates_args=(), device_types="cuda")
def maskedHadamardBwd_op(grad_flat: torch.Tensor, mask_bits: torch.Tensor, hadamard_matrix: torch.Tensor) -> torch.Tensor:
    """(g * mask).view(-1, hd) @ H^T with the mask given as bits (bit i of byte b = element 8b+i); an empty mask
    tensor means no mask.  [M,K] -> [M,K] of g's dtype."""
    g2 = _rows(grad_flat)
    return K.masked_hadamard_bwd(g2, hadamard_matrix.shape[0], g2.dtype, rotation_sign_bits(hadamard_matrix),
                                 mask_bits.contiguous() if mask_bits.numel() else None)


@maskedHadamardBwd_op.register_fake
def _(grad_flat, mask_bits, hadamard_matrix):
    return torch.empty_like(grad_flat)


def packed_forward(x2, weight, forward_matrix):
    """x [T,I], W [O,I] -> (y bf16 [T,O], packed operands kept for backward)."""
    xq, xs, xm = fusedQuantizeMx_op(x2, forward_matrix, True)
    wq, ws, wm = fusedQuantizeMx_op(weight, forward_matrix, True)
    y = matmul_mxf4_bf16_tn_op(xq, wq, xs, ws, constant_alpha(ALPHA_FWD, x2.device))
    return y, (xq, xs, xm, wq, ws, wm)


def packed_backward(e2, packed, forward_matrix, backward_matrix):
    """e [T,O] and the operands kept by packed_forward -> (grad x bf16 [T,I], grad W bf16 [O,I])."""
    xq, xs, xm, wq, ws, wm = packed
    one = constant_alpha(1.0, e2.device)
    alpha = constant_alpha(ALPHA_BWD, e2.device)
    eq, es = fusedQuantizeMxAbsMax_op(e2, backward_matrix, True)
    wtq, wts = backward_qt_bf16_op(wq, ws, backward_matrix, one)
    gx = maskedHadamardBwd_op(matmul_mxf4_bf16_tn_op(eq, wtq, es, wts, alpha), xm, forward_matrix)
    etq, ets = backward_t_bf16_op(e2, backward_matrix)
    xtq, xts = backward_qt_bf16_op(xq, xs, backward_matrix, one)
    gw = maskedHadamardBwd_op(matmul_mxf4_bf16_tn_op(etq, xtq, ets, xts, alpha), wm, forward_matrix)
    return gx, gw


class PackedLinearFn(torch.autograd.Function):
    """Quartet linear built from the operators above in the dataflow of the notebook's ``CudaGemm``: packed operands
    saved for backward, three FP4 products, masked inverse rotations.  ``forward_matrix`` rotates x and W,
    ``backward_matrix`` rotates the gradient-side operands (the caller re-randomises its signs between steps)."""

    @staticmethod
    def forward(ctx, input, weight, forward_matrix, backward_matrix):
        y, packed = packed_forward(input.flatten(end_dim=-2), weight, forward_matrix)
        ctx.save_for_backward(*packed, forward_matrix, backward_matrix)
        ctx.in_dtype, ctx.w_dtype = input.dtype, weight.dtype
        return y.view(*input.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, grad_output):
        *packed, hf, hb = ctx.saved_tensors
        gx, gw = packed_backward(grad_output.flatten(end_dim=-2).contiguous(), packed, hf, hb)
        return gx.view(*grad_output.shape[:-1], gx.shape[-1]).to(ctx.in_dtype), gw.to(ctx.w_dtype), None, None
