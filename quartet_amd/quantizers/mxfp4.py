"""MXFP4 quantizer modules with the reference's names, constructor kwargs and semantics
(src/models/quantization/quantizers/mxfp4.py), computed by the HIP kernels of libquartet_hip.so.

Differences in representation, not in results:
  * the rotation H = hd^-1/2 * Sylvester * diag(signs) is kept as a sign bit mask; the dense
    ``hadamard_matrix`` attribute is materialised on demand (same values the reference holds);
  * the clip mask saved for backward is bit-packed (1 bit per element);
  * ``rerotate="O32"`` replaces H by a dense random orthogonal matrix (mxfp4.py:61-64).  The kernels apply it on the
    matrix pipe (fp32 multiply-adds over the matrix rounded to the tensor's dtype, the role of the reference's
    in-kernel ``tl.dot``); a layer whose *gradient* quantizer holds a dense rotation stays on the packed FP4 path.
"""
import random
import weakref

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


_host_cache = {}
_HOST_CACHE_LIMIT = 64


def remember_host_value(kind, t, make):
    """Host-side value derived from tensor `t` (one device-to-host copy), kept while that very tensor object is alive
    and unmodified: the entry holds a weak reference, since an address alone may be handed to another tensor after a
    free."""
    key = (kind, id(t))
    hit = _host_cache.get(key)
    if hit is not None and hit[0]() is t and hit[1] == t._version:
        return hit[2]
    value = make()
    if len(_host_cache) >= _HOST_CACHE_LIMIT:
        _host_cache.clear()
    _host_cache[key] = (weakref.ref(t), t._version, value)
    return value


def register_host_value(kind, t, value):
    """Record a host-side value of tensor `t` that the caller already knows, so that remember_host_value finds it
    without a device-to-host copy."""
    if len(_host_cache) >= _HOST_CACHE_LIMIT:
        _host_cache.clear()
    _host_cache[(kind, id(t))] = (weakref.ref(t), t._version, value)


def sylvester_sign_bits(matrix):
    """Bit mask of the negated columns if `matrix` is ``hd^-1/2 * Sylvester * diag(+-1)`` (hd 32, 64 or 128, the
    scale rounded to the matrix's dtype), else None: a dense rotation."""
    if matrix.dim() != 2 or matrix.shape[0] != matrix.shape[1] or matrix.shape[0] not in (32, 64, 128):
        return None
    hd = matrix.shape[0]

    def read():
        h = matrix.detach().to("cpu", torch.float32)
        c = torch.tensor(hd ** -0.5, dtype=torch.float32).to(matrix.dtype).float()
        if not torch.equal(h, sylvester_matrix(hd) * c * torch.where(h[0] < 0, -1.0, 1.0)[None, :]):
            return -1
        return sum(1 << j for j, v in enumerate(h[0].tolist()) if v < 0)
    bits = remember_host_value("signs", matrix, read)
    return None if bits < 0 else bits


@torch.compiler.disable()
def mxfp4_forward_kernel_wrapper(x, hadamard_matrix, return_clip_mask=False, gaussian_scale=3 / 4,
                                 stochastic_round=False, quest=True):
    """Drop-in for mxfp4_triton.py:177-220: returns (pseudo-quantized tensor like x, bool clip mask | None).
    A signed, scaled Sylvester matrix (what the quantizer modules hold by default) runs on the butterfly kernels; any
    other matrix is applied as a dense matrix product and the kernel quantizes the rotated groups as they are."""
    hd = hadamard_matrix.shape[-1]
    mode = (K.QM_QUEST_SR if stochastic_round else K.QM_QUEST_RTN) if quest else \
        (K.QM_ABSMAX_SR if stochastic_round else K.QM_ABSMAX_RTN)
    seed = _fresh_seed() if stochastic_round else 0
    sign_bits = sylvester_sign_bits(hadamard_matrix)
    if sign_bits is None and hd == 32:
        _, _, mask, deq = K.quantize_mxfp4_dense(_as_2d(x, 32), hadamard_matrix, mode, seed=seed, want_mask=return_clip_mask,
                                                 want_dequant=True)
    elif sign_bits is None:   # a dense matrix of another size: library product, then the kernel quantizes the groups as they are
        _, _, mask, deq = K.quantize_mxfp4(_rotate_dense(x, hadamard_matrix), 1, None, mode, seed=seed,
                                           want_mask=return_clip_mask, want_dequant=True)
        deq = deq.to(x.dtype)
    else:
        _, _, mask, deq = K.quantize_mxfp4(_as_2d(x, hd), hd, sign_bits, mode, seed=seed, want_mask=return_clip_mask,
                                           want_dequant=True)
    clip = _unpack_mask(mask, x.shape).bool() if return_clip_mask else None
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
        self._dense = None  # fp32 [hd, hd] orthogonal matrix once re_randomize("O32") has replaced H
        self._dense_dev = None  # its copy on the device of the tensors being quantized
        self._dense_epoch = 0  # how many times re_randomize has drawn a dense matrix (keys a layer's cache of Q(W))
        self._matrix_dtype = torch.float32
        self._matrix_device = torch.device("cpu")

    @property
    def is_dense(self):
        return self._dense is not None

    @property
    def hadamard_matrix(self):
        hd = self.hadamard_dim
        if self._dense is not None:
            return self._dense.to(self._matrix_device).to(self._matrix_dtype)
        signs = torch.tensor([-1.0 if (self.sign_bits >> j) & 1 else 1.0 for j in range(hd)])
        h = sylvester_matrix(hd) * torch.tensor(hd ** -0.5, dtype=torch.float32) * signs[None, :]
        return h.to(self._matrix_device).to(self._matrix_dtype)

    def dense_matrix(self, device):
        """The dense rotation as the kernels read it (fp32 [32, 32] on `device`), or None while H is a signed Hadamard
        matrix.  Kept on the device until the next re_randomize replaces it."""
        if self._dense is None:
            return None
        if self._dense_dev is None or self._dense_dev.device != torch.device(device):
            self._dense_dev = self._dense.to(device=device, dtype=torch.float32).contiguous()
        return self._dense_dev

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
            # H <- U V^T of the SVD of a Gaussian matrix (mxfp4.py:61-64): Haar-distributed up to signs
            u, _, vh = torch.linalg.svd(torch.randn(self.hadamard_dim, self.hadamard_dim))
            self._dense = (u @ vh).contiguous()
            self._dense_dev = None
            self._dense_epoch += 1
            self.sign_bits = 0
        elif self.rerotate is None:
            pass
        else:
            raise ValueError(f"Invalid rerotate value: {self.rerotate}")


def _rotate_dense(x, matrix):
    """x.view(-1, hd) @ matrix with fp32 accumulation and an fp32 result, as rows of x's last dimension."""
    hd = matrix.shape[0]
    last = x.shape[-1] if x.dim() > 0 and x.shape[-1] % hd == 0 else hd
    return (x.reshape(-1, hd).float() @ matrix.to(x.dtype).float()).view(-1, last)


def _unpack_mask(maskbits, shape):
    shifts = torch.arange(8, device=maskbits.device, dtype=torch.uint8)
    return ((maskbits[..., None] >> shifts) & 1).view(shape)


class DenseRotationQuantizerFn(torch.autograd.Function):
    """Either quantizer with a dense rotation: for a 32 x 32 matrix the kernel rotates every group of 32 on the matrix
    pipe and quantizes it, a 64 x 64 or 128 x 128 matrix is applied as a library product first; straight-through backward ``(g * mask) @ matrix^T`` (mxfp4.py:30-34,143-146)."""

    @staticmethod
    def forward(ctx, x, matrix, mode, want_mask, post_scale):
        stochastic = mode in (K.QM_ABSMAX_SR, K.QM_QUEST_SR)
        seed = _fresh_seed() if stochastic else 0
        if matrix.shape[0] == 32:
            _, _, maskbits, deq = K.quantize_mxfp4_dense(_as_2d(x, 32), matrix, mode, seed=seed, want_mask=want_mask,
                                                         want_dequant=True)
        else:
            # a dense matrix over 64 or 128 values: library product in fp32, then the kernel quantizes the rotated groups
            # of 32 as they are (what mxfp4_forward_kernel_wrapper does for such a matrix)
            _, _, maskbits, deq = K.quantize_mxfp4(_rotate_dense(x, matrix), 1, None, mode, seed=seed, want_mask=want_mask,
                                                   want_dequant=True)
        if post_scale != 1.0:
            deq *= post_scale
        ctx.save_for_backward(matrix, maskbits) if want_mask else ctx.save_for_backward(matrix)
        ctx.x_shape, ctx.x_dtype, ctx.want_mask = x.shape, x.dtype, want_mask
        return deq.to(x.dtype).view(x.shape)

    @staticmethod
    def backward(ctx, grad_output):
        matrix = ctx.saved_tensors[0]
        g = grad_output
        if ctx.want_mask:
            g = g * _unpack_mask(ctx.saved_tensors[1], g.shape).to(g.dtype)
        out = g.reshape(-1, matrix.shape[0]) @ matrix.to(g.dtype).T
        return out.view(ctx.x_shape).to(ctx.x_dtype), None, None, None, None


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
        if self.is_dense:
            return DenseRotationQuantizerFn.apply(x, self.hadamard_matrix, K.QM_QUEST_RTN, True, 1.0)
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
        if self.is_dense:
            mode = K.QM_ABSMAX_SR if self.stochastic else K.QM_ABSMAX_RTN
            return DenseRotationQuantizerFn.apply(x, self.hadamard_matrix, mode, False, 1.0)
        return AlbertTsengQuantizerFn.apply(x, self.hadamard_dim, self.sign_bits, self.stochastic, 1.0)


class AlignedAlbertTsengQuantizer(_HadamardQuantizer):
    """mxfp4.py:71-124: absmax RTN with the output scaled by 1.009276."""

    def forward(self, x):
        self._note_input(x)
        if self.is_dense:
            return DenseRotationQuantizerFn.apply(x, self.hadamard_matrix, K.QM_ABSMAX_RTN, False, 1.009276)
        return AlbertTsengQuantizerFn.apply(x, self.hadamard_dim, self.sign_bits, False, 1.009276)
