"""MXFP4 quantizer modules with the reference's names, constructor kwargs and semantics
(src/models/quantization/quantizers/mxfp4.py), computed by the HIP kernels of libquartet_hip.so.

Differences in representation, not in results:
  * the rotation H = hd^-1/2 * Sylvester * diag(signs) is kept as a sign bit mask; the dense
    ``hadamard_matrix`` attribute is materialised on demand (same values the reference holds);
  * the clip mask saved for backward is bit-packed (1 bit per element);
  * ``rerotate="O32"`` (dense random rotation) is not built yet and raises.
"""
import random

import torch

from .. import kernels as K
from .base import BaseQuantizer


def sylvester_matrix(hd):
    """H[i,j] = (-1)^popcount(i&j): what hadamard_transform(eye(hd)) returns (mxfp4.py:42-44)."""
    idx = torch.arange(hd)
    bits = idx[:, None] & idx[None, :]
    pop = torch.zeros_like(bits)
    for b in range(8):
        pop += (bits >> b) & 1
    return torch.where(pop % 2 == 0, 1.0, -1.0)


def _fresh_seed():
    # one host-side draw per stochastic kernel launch, as mxfp4_triton.py:196-199 does
    return random.getrandbits(63)


def _as_2d(x, hd):
    """Contiguous 2-D view whose rows are whole Hadamard chunks; the kernel works on the flat
    buffer in chunks of hd (mxfp4_triton.py:39-44), so any such factorisation gives the same result."""
    x = x.contiguous()
    last = x.shape[-1] if x.dim() > 0 else 1
    if x.dim() >= 1 and last % hd == 0:
        return x.view(-1, last)
    return x.view(-1, hd)  # raises if numel is not a multiple of hd


def _autocast_bf16():
    return torch.is_autocast_enabled() and torch.get_autocast_dtype("cuda") == torch.bfloat16


@torch.compiler.disable()
def mxfp4_forward_kernel_wrapper(x, hadamard_matrix, return_clip_mask=False, gaussian_scale=3 / 4,
                                 stochastic_round=False, quest=True):
    """Drop-in for mxfp4_triton.py:177-220: returns (pseudo-quantized tensor like x, bool clip mask | None).
    ``hadamard_matrix`` must be a signed, scaled Sylvester matrix (what the quantizer modules hold)."""
    hd = hadamard_matrix.shape[-1]
    first = hadamard_matrix[0].float()
    sign_bits = 0
    for j, v in enumerate(first.tolist()):
        if v < 0:
            sign_bits |= 1 << j
    mode = (K.QM_QUEST_SR if stochastic_round else K.QM_QUEST_RTN) if quest else \
        (K.QM_ABSMAX_SR if stochastic_round else K.QM_ABSMAX_RTN)
    x2 = _as_2d(x, hd)
    _, _, mask, deq = K.quantize_mxfp4(x2, hd, sign_bits, mode, seed=_fresh_seed() if stochastic_round else 0,
                                       want_mask=return_clip_mask, want_dequant=True)
    clip = None
    if return_clip_mask:
        shifts = torch.arange(8, device=mask.device, dtype=torch.uint8)
        clip = ((mask[..., None] >> shifts) & 1).bool().view(x.shape)
    return deq.view(x.shape), clip


class _HadamardQuantizer(BaseQuantizer):
    """Shared state: Hadamard block size and the accumulated column signs of re_randomize."""

    def __init__(self, hadamard_dim=32, rerotate=None):
        super().__init__(4)
        if hadamard_dim not in (32, 64, 128):
            raise ValueError(f"hadamard_dim must be 32, 64 or 128, got {hadamard_dim}")
        self.hadamard_dim = hadamard_dim
        self.rerotate = rerotate
        self.sign_bits = 0  # bit j set = column j of H negated
        self._matrix_dtype = torch.float32
        self._matrix_device = torch.device("cpu")

    @property
    def hadamard_matrix(self):
        hd = self.hadamard_dim
        signs = torch.tensor([-1.0 if (self.sign_bits >> j) & 1 else 1.0 for j in range(hd)])
        h = sylvester_matrix(hd) * torch.tensor(hd ** -0.5, dtype=torch.float32) * signs[None, :]
        return h.to(self._matrix_device).to(self._matrix_dtype)

    def _note_input(self, x):
        # the reference re-casts its matrix to the input's device and dtype on every call (mxfp4.py:49,160)
        self._matrix_dtype, self._matrix_device = x.dtype, x.device

    def re_randomize(self):
        if self.rerotate == "signs":
            # H <- H @ diag(+-1) (mxfp4.py:53-60): flips accumulate, so they xor into the mask
            flips = torch.randint(0, 2, (self.hadamard_dim,))
            for j, f in enumerate(flips.tolist()):
                if f == 0:  # randint*2-1 == -1
                    self.sign_bits ^= 1 << j
        elif self.rerotate == "O32":
            raise NotImplementedError("rerotate='O32' (dense random orthogonal rotation) is not implemented")
        elif self.rerotate is None:
            pass
        else:
            raise ValueError(f"Invalid rerotate value: {self.rerotate}")


class QuestMXFP4QuantizerFn(torch.autograd.Function):
    """mxfp4.py:127-146: quest-scaled RTN forward with clip mask, masked straight-through backward."""

    @staticmethod
    def forward(ctx, x, hadamard_dim, sign_bits):
        x2 = _as_2d(x, hadamard_dim)
        _, _, maskbits, deq = K.quantize_mxfp4(x2, hadamard_dim, sign_bits, K.QM_QUEST_RTN, want_mask=True,
                                               want_dequant=True)
        ctx.save_for_backward(maskbits)
        ctx.hd, ctx.sign_bits, ctx.x_shape, ctx.x_dtype = hadamard_dim, sign_bits, x.shape, x.dtype
        return deq.view(x.shape)

    @staticmethod
    def backward(ctx, grad_output):
        (maskbits,) = ctx.saved_tensors
        g = grad_output.contiguous().view(maskbits.shape[0], -1)
        # under bf16 autocast the reference's `g @ H.T` runs with H cast to bf16 and a bf16 result
        low = _autocast_bf16() or g.dtype == torch.bfloat16
        sd = torch.bfloat16 if low else ctx.x_dtype
        out = K.masked_hadamard_bwd(g, ctx.hd, sd, ctx.sign_bits, maskbits, torch.bfloat16 if low else g.dtype)
        return out.view(ctx.x_shape).to(ctx.x_dtype), None, None


class QuestMXFP4Quantizer(_HadamardQuantizer):
    def forward(self, x):
        self._note_input(x)
        return QuestMXFP4QuantizerFn.apply(x, self.hadamard_dim, self.sign_bits)


class AlbertTsengQuantizerFn(torch.autograd.Function):
    """mxfp4.py:15-34: absmax/(3/4)-scaled RTN or SR forward, unmasked straight-through backward."""

    @staticmethod
    def forward(ctx, x, hadamard_dim, sign_bits, stochastic_round, post_scale):
        x2 = _as_2d(x, hadamard_dim)
        mode = K.QM_ABSMAX_SR if stochastic_round else K.QM_ABSMAX_RTN
        _, _, _, deq = K.quantize_mxfp4(x2, hadamard_dim, sign_bits, mode,
                                        seed=_fresh_seed() if stochastic_round else 0, want_dequant=True)
        if post_scale != 1.0:
            deq *= post_scale
        ctx.hd, ctx.sign_bits, ctx.x_shape, ctx.x_dtype = hadamard_dim, sign_bits, x.shape, x.dtype
        return deq.view(x.shape)

    @staticmethod
    def backward(ctx, grad_output):
        g = grad_output.contiguous().view(-1, ctx.x_shape[-1] if ctx.x_shape[-1] % ctx.hd == 0 else ctx.hd)
        low = _autocast_bf16() or g.dtype == torch.bfloat16
        sd = torch.bfloat16 if low else ctx.x_dtype
        out = K.masked_hadamard_bwd(g, ctx.hd, sd, ctx.sign_bits, None, torch.bfloat16 if low else g.dtype)
        return out.view(ctx.x_shape).to(ctx.x_dtype), None, None, None, None


class AlbertTsengQuantizer(_HadamardQuantizer):
    def __init__(self, hadamard_dim=32, stochastic=True, rerotate=None):
        super().__init__(hadamard_dim, rerotate)
        self.stochastic = stochastic

    def forward(self, x):
        self._note_input(x)
        return AlbertTsengQuantizerFn.apply(x, self.hadamard_dim, self.sign_bits, self.stochastic, 1.0)


class AlignedAlbertTsengQuantizer(_HadamardQuantizer):
    """mxfp4.py:71-124: absmax RTN with the output scaled by 1.009276."""

    def forward(self, x):
        self._note_input(x)
        return AlbertTsengQuantizerFn.apply(x, self.hadamard_dim, self.sign_bits, False, 1.009276)
