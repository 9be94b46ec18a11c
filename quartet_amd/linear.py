"""QuantizedLinear (API of the reference's src/models/quantization/__init__.py:11-42) and the fused
packed-MXFP4 autograd Function behind its production configuration.

Production configuration (main_setup.sh:77-93 of the reference): QuestMXFP4Quantizer on weights and
activations, AlbertTsengQuantizer on gradients, scheme "Q(E)Q(Wt)t_Q(Et)Q(Xt)t".  For it the layer
never materialises de-quantized tensors: operands stay packed (E2M1 codes + E8M0 scales + mask
bits, the tensors notebooks/benchmark_mxfp4.ipynb's CudaGemm saves) and the three products run on
the block-scaled FP4 MFMA.  Any other mix of quantizers/schemes takes the generic path through the
quantizer modules and library GEMMs, as the reference does."""
import torch
import torch.nn as nn

from . import _lib
from . import kernels as K
from .backward import BACKWARD_SCHEMES, EW_EtX_Scheme, QEQWtt_QEtQXtt_Scheme  # noqa: F401
from .quantizers import QUANTIZER_CLASSES, AlbertTsengQuantizer, NoQuantizer, QuestMXFP4Quantizer  # noqa: F401
from .quantizers.mxfp4 import _autocast_bf16, _fresh_seed


_SEED_BASE = None


def set_device_seed_base(tensor):
    """A one-element int64 tensor on the GPU (or None to switch this off) whose value the gradient quantizers of every
    packed-path layer add to their seeds when their kernels run.  The reference draws a fresh host seed per stochastic
    quantization (mxfp4_triton.py:196-199); a training step replayed from a captured HIP graph would repeat the seeds
    drawn at capture time, so capture the step with a seed base set and let the graph increment the tensor (any
    in-place add recorded in the graph): every replay then rounds with fresh random streams.  The sign flips drawn at
    capture time stay as they are.  Applies to layers on the tiled layout (tokens, in- and out-features multiples of
    128, Hadamard blocks 32, no dense rotation); a stochastic layer outside it raises while a seed base is set, since
    its replays would repeat their random streams."""
    global _SEED_BASE
    if tensor is not None and not (tensor.is_cuda and tensor.dtype == torch.int64 and tensor.numel() >= 1):
        raise ValueError("the seed base must be an int64 tensor on the GPU")
    _SEED_BASE = tensor


def _use_tiled_codes(T, I, O, a_q, w_q, g_q):
    """Tiled code bytes (16 rows x 128 elements contiguous) when every operand of the three products qualifies: all
    three extents multiples of 128 and at least 256, Hadamard block 32 throughout; row-major codes otherwise."""
    return (all(d % 128 == 0 and d >= 256 for d in (T, I, O)) and
            a_q.hadamard_dim == 32 and w_q.hadamard_dim == 32 and g_q.hadamard_dim == 32)


def _forward_packed(ctx, x2, weight, a_q, w_q, g_q, weight_cache, tiled, out_dtype, x_dtype, packed_x=None, rows=None):
    """F1 (unless a producer already wrote packed_x), F2 (unless the layer's cache holds Q(W)), F3; records on ctx what
    the backward pass of the products needs.  Returns (y [T, O], packed_x, packed_w)."""
    w2 = weight.contiguous()
    # a forward quantizer that holds the dense matrix of rerotate="O32": its kernel fills the packed operand here, and the
    # straight-through backward (clip mask, transposed matrix) is applied to the rotated-basis gradient in _backward_packed
    # (the matrix cast to the quantized tensor's dtype as the quantizer modules do, mxfp4.py:49,160; fp32 storage for the kernel)
    x_dense = a_q.dense_matrix(w2.device).to(x_dtype).to(torch.float32) if a_q.is_dense else None
    w_dense = w_q.dense_matrix(w2.device).to(w2.dtype).to(torch.float32) if w_q.is_dense else None
    if x_dense is not None and packed_x is None:
        packed_x, rows, x2 = K.quantize_dense_into_packed(x2, x_dense, tiled), x2.shape[0], None
    # Q(W) of an unchanged weight (the micro-steps of one accumulation) is quantized once and kept by the layer
    key = (weight.data_ptr(), weight._version, weight.dtype, tuple(weight.shape), w_q.hadamard_dim, w_q.sign_bits, tiled,
           None if w_dense is None else w_q._dense_epoch)
    packed_w = weight_cache.get(key) if weight_cache is not None else None
    if w_dense is not None and packed_w is None:
        packed_w = K.quantize_dense_into_packed(w2, w_dense, tiled)
    y, packed_x, packed_w = K.linear_forward(x2, w2, a_q.hadamard_dim, a_q.sign_bits, w_q.hadamard_dim, w_q.sign_bits,
                                             out_dtype, tiled, packed_w, packed_x, rows)
    if weight_cache is not None:
        weight_cache.put(key, packed_w)
    ctx.g_q = g_q
    ctx.tiled = tiled
    ctx.dense_fwd = (x_dense, w_dense)
    ctx.fwd = (a_q.hadamard_dim, a_q.sign_bits, w_q.hadamard_dim, w_q.sign_bits)
    ctx.dims = (y.shape[0], weight.shape[1], weight.shape[0])
    ctx.x_dtype, ctx.w_dtype = x_dtype, weight.dtype
    return y, packed_x, packed_w


def _dense_rotation_backward(g, maskbits, matrix, scale_dtype):
    """Straight-through backward of a forward quantizer with a dense rotation (mxfp4.py:143-146 with the matrix of
    mxfp4.py:61-64): (g * clip mask) @ matrix^T per group of 32, in g's dtype like the module path's product."""
    from .quantizers.mxfp4 import _unpack_mask
    g = g * _unpack_mask(maskbits, g.shape).to(g.dtype)
    m = matrix.to(scale_dtype).to(g.dtype)
    return (g.reshape(-1, 32) @ m.T).view(g.shape)


def _backward_packed(ctx, e, packed_x, packed_w, gx_rotated=False):
    """B1-B8: e [.., O] -> (gradient w.r.t. the tensor F1 quantized [T, I], gradient w.r.t. W [O, I]).  With
    `gx_rotated` B7 is left out: returns (gradient in F1's rotated basis, gradient w.r.t. W, (mask bits, signs, scale
    dtype) that the consumer's kernel needs to apply B7 itself)."""
    g_q = ctx.g_q
    a_hd, a_signs, w_hd, w_signs = ctx.fwd
    T, I, O = ctx.dims
    g_q.re_randomize()
    hd, signs = g_q.hadamard_dim, g_q.sign_bits
    # rerotate="O32": the four gradient quantizations rotate by the dense matrix drawn just now, on the matrix pipe
    g_matrix = g_q.dense_matrix(e.device) if g_q.is_dense else None
    mode = K.QM_ABSMAX_SR if g_q.stochastic else K.QM_ABSMAX_RTN
    # one host-side draw per stochastic quantization, in the order e, W^T, e^T, x^T
    seeds = [_fresh_seed() if g_q.stochastic else 0 for _ in range(4)]
    e2 = e.reshape(-1, e.shape[-1]).contiguous()
    low = _autocast_bf16() or e2.dtype == torch.bfloat16
    mid_dtype = torch.bfloat16 if low else e2.dtype
    sd_x = torch.bfloat16 if low else ctx.x_dtype
    sd_w = torch.bfloat16 if low else ctx.w_dtype
    if _SEED_BASE is not None and g_q.stochastic and not (ctx.tiled and g_matrix is None):
        # the device seed base is read by the pair launches of the tiled layout only: on any other path a captured replay
        # would silently repeat this launch's random streams
        raise _lib.QuartetHipError(
            f"a device seed base is set (set_device_seed_base), but this layer (tokens {T}, in {I}, out {O}"
            f"{', dense gradient rotation' if g_matrix is not None else ''}) does not run on the tiled layout, whose kernels are the "
            "only ones that read it (every extent a multiple of 128 and >= 256, Hadamard blocks 32, no dense rotation); "
            "clear the seed base or change the layer")
    x_dense, w_dense = ctx.dense_fwd
    gx, gw = K.linear_backward(e2, packed_x, packed_w, T, I, O, a_hd, a_signs, w_hd, w_signs, hd, signs, mode, seeds, ctx.x_dtype,
                               ctx.w_dtype, mid_dtype, sd_x, sd_w, ctx.tiled, gx_rotated or x_dense is not None,
                               ctx.w_dtype if ctx.w_dtype in (torch.float32, torch.bfloat16) else None, g_matrix,
                               _SEED_BASE if (ctx.tiled and g_matrix is None and g_q.stochastic) else None,
                               gw_rotated=w_dense is not None)
    if w_dense is not None:
        gw = _dense_rotation_backward(gw, K.packed_mask_bits(packed_w, O, I), w_dense, sd_w)
    if gx_rotated:
        assert x_dense is None   # the fused producers are not offered layers with a dense forward rotation
        return gx, gw, (K.packed_mask_bits(packed_x, T, I), a_signs, sd_x)
    if x_dense is not None:
        gx = _dense_rotation_backward(gx, K.packed_mask_bits(packed_x, T, I), x_dense, sd_x)
    return gx, gw


class QuartetLinearFn(torch.autograd.Function):
    """y = Q(x) Q(W)^T with the fully quantized backward of backward.py:57-85, on packed operands.

    forward : F1/F2 quantize (quest RTN + mask) -> F3 FP4 GEMM
    backward: re-randomise signs; B1 Q(e); B2 Q(Q(W)^T); B3 GEMM -> grad wrt Q(x);
              B4 Q(e^T); B5 Q(Q(x)^T); B6 GEMM -> grad wrt Q(W);
              B7/B8 masked inverse rotation (straight-through estimators of F1/F2)."""

    @staticmethod
    def forward(ctx, x, weight, a_q, w_q, g_q, weight_cache):
        in_features = weight.shape[1]
        x2 = x.reshape(-1, in_features).contiguous()
        out_dtype = torch.bfloat16 if _autocast_bf16() else x.dtype
        tiled = _use_tiled_codes(x2.shape[0], in_features, weight.shape[0], a_q, w_q, g_q)
        y, packed_x, packed_w = _forward_packed(ctx, x2, weight, a_q, w_q, g_q, weight_cache, tiled, out_dtype, x.dtype)
        ctx.save_for_backward(packed_x, packed_w)
        ctx.x_shape = x.shape
        return y.view(*x.shape[:-1], weight.shape[0])

    @staticmethod
    def backward(ctx, e):
        packed_x, packed_w = ctx.saved_tensors
        gx, gw = _backward_packed(ctx, e, packed_x, packed_w)
        return gx.to(ctx.x_dtype).view(ctx.x_shape), gw.to(ctx.w_dtype), None, None, None, None


class PackedWeightCache:
    """The packed Q(W) of a layer's current weight, kept across the micro-steps of one gradient accumulation (the
    weight changes only at the optimizer step, src/optim/base.py:188-207 of the reference).  One entry, replaced --
    never overwritten in place, so that a graph built earlier keeps the buffer it saved -- when the weight's storage,
    version counter, rotation or code layout changes.  An update that bypasses the version counter (``weight.data``
    arithmetic) is invisible to the key: whoever steps the optimizer calls ``invalidate_packed_weights`` afterwards,
    as ``quartet_amd.train.train`` does, and the cache is off unless ``enable_packed_weight_cache`` turned it on."""

    def __init__(self):
        self.key, self.buffer, self.hits, self.misses = None, None, 0, 0

    def get(self, key):
        if key == self.key:
            self.hits += 1
            return self.buffer
        self.misses += 1
        return None

    def put(self, key, buffer):
        self.key, self.buffer = key, buffer

    def clear(self):
        self.key, self.buffer = None, None


def enable_packed_weight_cache(model, enabled=True):
    """Give every QuantizedLinear of `model` a PackedWeightCache (or remove it)."""
    for m in model.modules():
        if isinstance(m, QuantizedLinear):
            m.packed_weight_cache = PackedWeightCache() if enabled else None


def invalidate_packed_weights(model):
    """Forget every cached Q(W): call after anything that changes the weights (the optimizer step)."""
    for m in model.modules():
        if isinstance(m, QuantizedLinear) and m.packed_weight_cache is not None:
            m.packed_weight_cache.clear()


class QuantizedLinear(nn.Linear):
    """nn.Linear whose forward is scheme(act_q(x), weight_q(W)); the bias parameter, if requested,
    is never applied -- exactly as in the reference (the scheme calls F.linear(x, w, None))."""

    def __init__(self, in_features, out_features, weight_quantizer=None, activation_quantizer=None,
                 gradient_quantizer=None, backward_scheme=None, **kwargs):
        super().__init__(in_features, out_features, **kwargs)
        if weight_quantizer is None:
            weight_quantizer = NoQuantizer()
        if activation_quantizer is None:
            activation_quantizer = NoQuantizer()
        if gradient_quantizer is None:
            gradient_quantizer = NoQuantizer()
        if backward_scheme is None:
            backward_scheme = EW_EtX_Scheme()
        self.weight_quantizer = weight_quantizer
        self.activation_quantizer = activation_quantizer
        self.backward_scheme = backward_scheme
        self.backward_scheme.g_quantizer = gradient_quantizer
        self.use_packed_path = True
        self.packed_weight_cache = None  # see enable_packed_weight_cache

    def _is_production_config(self, tokens):
        g_q = self.backward_scheme.g_quantizer
        # A dense rotation (rerotate="O32") replaces a Hadamard block of 32 only in the kernels.  In the gradient quantizer
        # the packed path serves it when every extent is a multiple of 128; in a forward quantizer (the reference's loop
        # never re-randomises those) the dense quantizer kernel fills the packed operand and the straight-through
        # backward is a small library product.
        dense = any(getattr(q_, "is_dense", False) and q_.hadamard_dim != 32
                    for q_ in (self.activation_quantizer, self.weight_quantizer))
        if getattr(g_q, "is_dense", False) or getattr(g_q, "rerotate", None) == "O32":
            dense = dense or g_q.hadamard_dim != 32 or any(d % 128 for d in (tokens, self.in_features, self.out_features))
        return (self.use_packed_path and not dense
                and type(self.activation_quantizer) is QuestMXFP4Quantizer
                and type(self.weight_quantizer) is QuestMXFP4Quantizer
                and type(g_q) is AlbertTsengQuantizer
                and type(self.backward_scheme) is QEQWtt_QEtQXtt_Scheme)

    def forward(self, x):
        if self._is_production_config(x.numel() // max(x.shape[-1], 1)):
            return QuartetLinearFn.apply(x, self.weight, self.activation_quantizer, self.weight_quantizer,
                                         self.backward_scheme.g_quantizer, self.packed_weight_cache)
        xq = self.activation_quantizer(x)
        wq = self.weight_quantizer(self.weight)
        return self.backward_scheme(xq, wq)
