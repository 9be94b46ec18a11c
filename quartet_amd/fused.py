"""Producers fused into the activation quantizer of a Quartet linear.

In the model the quantized linears sit in (src/models/llama.py of the reference) two of the four linears of a block are
fed by RMSNorm (``c_attn(ln_1(x))``, ``w12(ln_2(x))``, llama.py:170-171) and one by the SwiGLU product
(``c_proj(silu(up) * gate)``, llama.py:113-114).  ``rmsnorm_linear`` and ``swiglu_linear`` compute the same results
without writing the normalised tensor / the product: the quantizer kernel builds each group of 32 values in registers,
the layer consumes the packed operand, and the backward pass recomputes what it needs from the producer's inputs.

Both fall back to the unfused composition (same mathematics, more memory traffic) when the layer is not in its
production configuration, uses another Hadamard block than 32, or the tensors are not what the kernels take."""
import torch
import torch.nn.functional as F

from . import kernels as K
from .linear import QuantizedLinear, _backward_packed, _forward_packed, _use_tiled_codes
from .quantizers.mxfp4 import _autocast_bf16

_KERNEL_DTYPES = (torch.float32, torch.bfloat16)


def _layer_is_fusable(layer, x):
    return (isinstance(layer, QuantizedLinear) and layer._is_production_config(x.numel() // max(x.shape[-1], 1)) and layer.weight.is_cuda
            and layer.activation_quantizer.hadamard_dim == 32 and not layer.activation_quantizer.is_dense
            and layer.weight.dtype in _KERNEL_DTYPES)


class RMSNormLinearFn(torch.autograd.Function):
    """y = Q(rmsnorm(x) * gain) Q(W)^T; backward = the layer's quantized backward followed by RMSNorm's.

    With `pass_input` the function also returns x itself: a block computes ``x + f(norm(x))``, and when the residual sum
    takes this second output instead of x, both gradients of x (through the norm and past it) arrive here together and
    the RMSNorm backward kernel adds them, instead of autograd in a pass of its own.  With `add` (x fp32) the norm's
    input is ``x + add``, formed inside the quantizer kernel; the sum is the second output."""

    @staticmethod
    def forward(ctx, x, add, gain, weight, eps, a_q, w_q, g_q, weight_cache, pass_input=False):
        I = weight.shape[1]
        x2 = x.reshape(-1, I).contiguous()
        T, O = x2.shape[0], weight.shape[0]
        tiled = _use_tiled_codes(T, I, O, a_q, w_q, g_q)
        if add is None:
            packed_x, factor = K.rmsnorm_quantize(x2, gain, eps, a_q.sign_bits, tiled)
        else:
            packed_x, factor, x2 = K.rmsnorm_quantize(x2, gain, eps, a_q.sign_bits, tiled, add.reshape(-1, I).contiguous())
        # the normalised tensor times the fp32 gain is an fp32 tensor: that is the dtype the layer sees
        out_dtype = torch.bfloat16 if _autocast_bf16() else torch.float32
        y, packed_x, packed_w = _forward_packed(ctx, None, weight, a_q, w_q, g_q, weight_cache, tiled, out_dtype, torch.float32,
                                                packed_x, T)
        ctx.save_for_backward(x2, gain, factor, packed_x, packed_w)
        ctx.x_shape = x.shape
        ctx.add_dtype = None if add is None else add.dtype
        y = y.view(*x.shape[:-1], O)
        if add is not None:
            return y, x2.view(x.shape)
        return (y, x) if pass_input else y

    @staticmethod
    def backward(ctx, e, skip=None):
        x2, gain, factor, packed_x, packed_w = ctx.saved_tensors
        # B7 (the quantizer's straight-through backward) runs inside the RMSNorm backward kernel
        gy, gw, (maskbits, signs, scale_dtype) = _backward_packed(ctx, e, packed_x, packed_w, gx_rotated=True)
        if skip is not None:
            skip = skip.reshape(x2.shape).to(x2.dtype).contiguous()
        want_copy = ctx.add_dtype == torch.bfloat16
        out = K.rmsnorm_backward(gy, x2, gain, factor, maskbits, signs, scale_dtype, skip, want_copy)
        dx = out[0].view(ctx.x_shape)
        d_add = None if ctx.add_dtype is None else (out[2].view(ctx.x_shape) if want_copy else dx)
        return dx, d_add, out[1], gw.to(ctx.w_dtype), None, None, None, None, None, None


class SwiGLULinearFn(torch.autograd.Function):
    """y = Q(silu(up) * gate) Q(W)^T with h12 = (up, gate); backward = the layer's quantized backward, then SwiGLU's."""

    @staticmethod
    def forward(ctx, h12, weight, a_q, w_q, g_q, weight_cache):
        I = weight.shape[1]
        h2 = h12.reshape(-1, 2 * I).contiguous()
        T, O = h2.shape[0], weight.shape[0]
        tiled = _use_tiled_codes(T, I, O, a_q, w_q, g_q)
        packed_x = K.swiglu_quantize(h2, a_q.sign_bits, tiled)
        out_dtype = torch.bfloat16 if _autocast_bf16() else h12.dtype
        y, packed_x, packed_w = _forward_packed(ctx, None, weight, a_q, w_q, g_q, weight_cache, tiled, out_dtype, h12.dtype,
                                                packed_x, T)
        ctx.save_for_backward(h2, packed_x, packed_w)
        ctx.h_shape = h12.shape
        return y.view(*h12.shape[:-1], O)

    @staticmethod
    def backward(ctx, e):
        h2, packed_x, packed_w = ctx.saved_tensors
        g, gw, (maskbits, signs, scale_dtype) = _backward_packed(ctx, e, packed_x, packed_w, gx_rotated=True)
        d_h12 = K.swiglu_backward(g, h2, maskbits, signs, scale_dtype)
        return d_h12.view(ctx.h_shape), gw.to(ctx.w_dtype), None, None, None, None


class RopeQKVFn(torch.autograd.Function):
    """(q, k, v) [B, T, heads, head_dim] from the fused projection [B, T, 3C]: q and k rotated (llama.py:43-61), all three
    in the dtype attention will run in, in one pass; backward merges the three gradients into [B, T, 3C]."""

    @staticmethod
    def forward(ctx, qkv, table, n_head):
        B, T, C3 = qkv.shape
        C = C3 // 3
        hs = C // n_head
        # the reference rotates in fp32 and autocast hands attention bf16 copies: one rounding of the fp32 result
        out_dtype = torch.bfloat16 if _autocast_bf16() else torch.float32
        q, k, v = K.rope_split_qkv(qkv.reshape(B * T, C3).contiguous(), table, C, hs, T, out_dtype)
        ctx.save_for_backward(table)
        ctx.meta = (B, T, C, n_head, hs, qkv.dtype)
        return q.view(B, T, n_head, hs), k.view(B, T, n_head, hs), v.view(B, T, n_head, hs)

    @staticmethod
    def backward(ctx, dq, dk, dv):
        (table,) = ctx.saved_tensors
        B, T, C, n_head, hs, in_dtype = ctx.meta
        dt = dq.dtype
        flat = lambda g: g.to(dt).contiguous().view(B * T, C)
        d_qkv = K.rope_merge_qkv_grad(flat(dq), flat(dk), flat(dv), table, C, hs, T, in_dtype)
        return d_qkv.view(B, T, 3 * C), None, None


def rope_qkv(qkv, table, n_head):
    """Split the fused attention projection [B, T, 3C] into q, k, v [B, T, n_head, head_dim] with q and k rotated by the
    (cos, sin) table [T, head_dim/2, 2]."""
    C = qkv.shape[-1] // 3
    hs = C // n_head
    if qkv.is_cuda and qkv.dtype in _KERNEL_DTYPES and hs % 8 == 0 and table.dtype == torch.float32:
        return RopeQKVFn.apply(qkv, table.contiguous(), n_head)
    from .llama import apply_rotary
    B, T, _ = qkv.shape
    q, k, v = qkv.split(C, dim=2)
    q, k = apply_rotary(q.view(B, T, n_head, hs), k.view(B, T, n_head, hs), table)
    return q, k, v.view(B, T, n_head, hs)


def rmsnorm_linear(norm, layer, x, pass_input=False, add=None):
    """layer(norm(x)) for an RMSNorm module `norm` (attributes ``weight`` and ``eps``) and a QuantizedLinear.  With
    `pass_input` returns (layer(norm(x)), x): use the second value for the residual sum around the norm, so that the sum
    of x's two gradients happens inside the RMSNorm backward kernel.  With `add` returns (layer(norm(x + add)), x + add):
    the residual sum in front of the norm is formed inside the quantizer kernel."""
    fusable = (_layer_is_fusable(layer, x) and x.is_cuda and x.dtype in _KERNEL_DTYPES and norm.weight.dtype == torch.float32
               and x.shape[-1] <= 8192)
    if fusable and add is not None and not (x.dtype == torch.float32 and add.dtype in _KERNEL_DTYPES and add.shape == x.shape):
        x, add = x + add, None
        pass_input = True
    if fusable:
        return RMSNormLinearFn.apply(x, add, norm.weight, layer.weight, norm.eps, layer.activation_quantizer, layer.weight_quantizer,
                                     layer.backward_scheme.g_quantizer, layer.packed_weight_cache, pass_input)
    if add is not None:
        x = x + add
    y = layer(norm(x))
    return (y, x) if (pass_input or add is not None) else y


def swiglu_linear(layer, h12):
    """layer(silu(up) * gate) with (up, gate) the two halves of h12's last dimension."""
    if _layer_is_fusable(layer, h12) and h12.is_cuda and h12.dtype in _KERNEL_DTYPES:
        return SwiGLULinearFn.apply(h12, layer.weight, layer.activation_quantizer, layer.weight_quantizer,
                                    layer.backward_scheme.g_quantizer, layer.packed_weight_cache)
    up, gate = h12.split(h12.shape[-1] // 2, dim=-1)
    return layer(F.silu(up) * gate)
