"""Backward schemes: which operands of a linear layer's two gradient products are quantized.

Registry keys, class names and operand orientation follow the reference's
src/models/quantization/backward.py; these generic schemes work on the pseudo-quantized (de-quantized)
tensors the quantizer modules return and use library GEMMs, except that the error-only scheme multiplies the *packed*
Q(e) with the saved bf16 operands in this build's own FP4 x bf16 kernel whenever its products run in bf16.  The production
combination never gets here: ``quartet_amd.linear`` routes it to the packed-FP4 path.

For y = x W^T with upstream gradient e (tokens flattened to rows):

    scheme key                  grad_x                   grad_W                     sign re-randomisation
    EW_EtX                      e W                      e^T x                      -
    Q(E)W_Q(Et)X                Q(e) W                   Q(e^T) x                   -
    Q(E)Q(Wt)t_Q(Et)Q(Xt)t      Q(e) Q(W^T)^T            Q(e^T) Q(x^T)^T            once, before the four Q(.)

Every Q(.) quantizes along its tensor's last axis, which is the contraction axis of the product it feeds,
hence the explicit transposes."""
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd import Function

from . import kernels as K
from .quantizers.mxfp4 import (AlbertTsengQuantizer, AlignedAlbertTsengQuantizer, QuestMXFP4Quantizer, _autocast_bf16,
                               _fresh_seed)


def _save_and_multiply(ctx, x, w, g_quantizer):
    ctx.save_for_backward(x, w)
    ctx.g_quantizer = g_quantizer
    return F.linear(x, w, None)


def _packed_error_products(q, e_rows, w, x_rows):
    """grad_x = Q(e) w and grad_w = Q(e^T) x on the packed codes of Q(e), Q(e^T) (qm_gemm_mxfp4_bf16_nn): no de-quantized
    copy of the error signal, no transposed copy of e.  Serves the MXFP4 quantizers with a Hadamard rotation when the
    products run in bf16 (bf16 autocast, or bf16 tensors throughout) on the GPU; returns None for anything else, which
    then takes the module path below.  What differs from that path: the de-quantized Q(e) is not rounded to bf16 before
    the product (codes times scale are exact in bf16; the factor 4/3 of the absmax modes is applied to the fp32 sums)."""
    if not isinstance(q, (AlbertTsengQuantizer, AlignedAlbertTsengQuantizer, QuestMXFP4Quantizer)) or q.is_dense:
        return None
    if not (e_rows.is_cuda and w.is_cuda and x_rows.is_cuda):
        return None
    low = _autocast_bf16() or (e_rows.dtype == w.dtype == x_rows.dtype == torch.bfloat16)
    if not low or e_rows.dtype not in (torch.bfloat16, torch.float32):
        return None
    T, O = e_rows.shape
    I = w.shape[1]
    hd = q.hadamard_dim
    if not (K.gemm_mxfp4_bf16_nn_supported(T, I, O) and K.gemm_mxfp4_bf16_nn_supported(O, I, T)) or O % hd or T % hd or T % 8:
        return None
    if isinstance(q, QuestMXFP4Quantizer):
        mode, alpha = K.QM_QUEST_RTN, 1.0
    elif isinstance(q, AlignedAlbertTsengQuantizer):
        mode, alpha = K.QM_ABSMAX_RTN, K.FOUR_THIRDS * 1.009276
    else:
        mode, alpha = (K.QM_ABSMAX_SR if q.stochastic else K.QM_ABSMAX_RTN), K.FOUR_THIRDS
    stochastic = mode == K.QM_ABSMAX_SR
    q._note_input(e_rows)
    e2 = e_rows.contiguous()
    ec, es, _, _ = K.quantize_mxfp4(e2, hd, q.sign_bits, mode, seed=_fresh_seed() if stochastic else 0)
    grad_x = K.gemm_mxfp4_bf16_nn(ec, es, w.to(torch.bfloat16).contiguous(), alpha, torch.bfloat16)
    etc, ets, _, _ = K.quantize_mxfp4(e2, hd, q.sign_bits, mode, transposed_in=True, seed=_fresh_seed() if stochastic else 0)
    grad_w = K.gemm_mxfp4_bf16_nn(etc, ets, x_rows.to(torch.bfloat16).contiguous(), alpha, torch.bfloat16)
    return grad_x, grad_w


def _gradients(ctx, e, quantize_saved):
    """The two gradient products with the gradient quantizer applied to e (always) and, when
    ``quantize_saved``, to the saved operands as well."""
    x, w = ctx.saved_tensors
    q = ctx.g_quantizer
    out_features, in_features = w.shape
    x_rows = x.reshape(-1, in_features)
    e_rows = e.reshape(-1, out_features)
    if quantize_saved:
        q.re_randomize()
        grad_x = q(e) @ q(w.T.contiguous()).T
        grad_w = q(e_rows.T.contiguous()) @ q(x_rows.T.contiguous()).T
    else:
        packed = _packed_error_products(q, e_rows, w, x_rows)
        if packed is not None:
            return packed[0].view(*e.shape[:-1], in_features), packed[1], None
        grad_x = q(e) @ w
        grad_w = q(e_rows.T.contiguous()) @ x_rows
    return grad_x, grad_w, None


class QEW_QEtXFn(Function):
    """backward.py:21-45: only the error signal is quantized."""

    @staticmethod
    def forward(ctx, x, w, g_quantizer):
        return _save_and_multiply(ctx, x, w, g_quantizer)

    @staticmethod
    def backward(ctx, e):
        return _gradients(ctx, e, quantize_saved=False)


class QEQWtt_QEtQXttFn(Function):
    """backward.py:57-85: all four operands of the gradient products are quantized."""

    @staticmethod
    def forward(ctx, x, w, g_quantizer):
        return _save_and_multiply(ctx, x, w, g_quantizer)

    @staticmethod
    def backward(ctx, e):
        return _gradients(ctx, e, quantize_saved=True)


class EW_EtX_Scheme(nn.Module):
    """No quantization in backward; ``g_quantizer`` is attached by QuantizedLinear and unused here."""

    fn = None

    def __init__(self):
        super().__init__()
        self.g_quantizer = None

    def forward(self, x, w):
        if self.fn is None:
            return F.linear(x, w, None)
        return self.fn.apply(x, w, self.g_quantizer)


class QEW_QEtX_Scheme(EW_EtX_Scheme):
    fn = QEW_QEtXFn


class QEQWtt_QEtQXtt_Scheme(QEW_QEtX_Scheme):
    fn = QEQWtt_QEtQXttFn


BACKWARD_SCHEMES = {
    "EW_EtX": EW_EtX_Scheme,
    "Q(E)W_Q(Et)X": QEW_QEtX_Scheme,
    "Q(E)Q(Wt)t_Q(Et)Q(Xt)t": QEQWtt_QEtQXtt_Scheme,
}
