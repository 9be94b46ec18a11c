"""Backward schemes: which operands of a linear layer's two gradient products are quantized.

Registry keys, class names and operand orientation follow the reference's
src/models/quantization/backward.py; these generic schemes work on the pseudo-quantized (de-quantized)
tensors the quantizer modules return and use library GEMMs.  The production combination never gets here:
``quartet_amd.linear`` routes it to the packed-FP4 path.

For y = x W^T with upstream gradient e (tokens flattened to rows):

    scheme key                  grad_x                   grad_W                     sign re-randomisation
    EW_EtX                      e W                      e^T x                      -
    Q(E)W_Q(Et)X                Q(e) W                   Q(e^T) x                   -
    Q(E)Q(Wt)t_Q(Et)Q(Xt)t      Q(e) Q(W^T)^T            Q(e^T) Q(x^T)^T            once, before the four Q(.)

Every Q(.) quantizes along its tensor's last axis, which is the contraction axis of the product it feeds,
hence the explicit transposes."""
import torch.nn as nn
import torch.nn.functional as F
from torch.autograd import Function


def _save_and_multiply(ctx, x, w, g_quantizer):
    ctx.save_for_backward(x, w)
    ctx.g_quantizer = g_quantizer
    return F.linear(x, w, None)


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
