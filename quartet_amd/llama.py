"""The Llama-style model the Quartet linears sit in: the caller of the quantized-linear path.

Structure, parameter names and numerics follow the reference's src/models/llama.py:78-262 and
src/models/base.py:33-78,229-235: pre-norm blocks ``x + attn(ln_1 x)``, ``x + mlp(ln_2 x)``; a fused
``c_attn`` (d -> 3d) and ``c_proj`` per attention; SwiGLU with a fused ``w12`` (d -> 2 d_ff, split order
*up then gate*) and ``c_proj``; interleaved-pair rotary embedding evaluated in fp32 (theta 1e4);
RMSNorm in fp32; causal scaled-dot-product attention; untied, unquantized ``lm_head``; every block
linear is a ``QuantizedLinear`` built from registry names; init N(0, init_std) with ``c_proj`` weights at
``init_std / sqrt(2 n_layer)``; cross-entropy over all positions.  The tokenizer the reference attaches
(tiktoken) is not part of the numerics and is left out.

Everything here except the block linears is stock PyTorch: this module is plumbing around the hot path."""
import contextlib
import math
from dataclasses import dataclass, field

import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.nn.attention import SDPBackend, sdpa_kernel

from .backward import BACKWARD_SCHEMES
from .fused import rmsnorm_linear, rope_qkv, swiglu_linear
from .linear import QuantizedLinear
from .quantizers import QUANTIZER_CLASSES


@dataclass
class LlamaConfig:
    """Fields and defaults of the reference's argparse config (src/config/base.py) that the model reads."""
    vocab_size: int = 32000
    sequence_length: int = 512
    n_layer: int = 6
    n_head: int = 5
    n_embd: int = 640
    multiple_of: int = 256
    rmsnorm_eps: float = 1e-5
    dropout: float = 0.0
    bias: bool = False
    init_std: float = 0.02
    w_quant: str = "QuestMXFP4Quantizer"
    w_quant_kwargs: dict = field(default_factory=lambda: {"hadamard_dim": 32})
    a_quant: str = "QuestMXFP4Quantizer"
    a_quant_kwargs: dict = field(default_factory=lambda: {"hadamard_dim": 32})
    g_quant: str = "AlbertTsengQuantizer"
    g_quant_kwargs: dict = field(default_factory=lambda: {"hadamard_dim": 32, "stochastic": True, "rerotate": "signs"})
    backward_scheme: str = "Q(E)Q(Wt)t_Q(Et)Q(Xt)t"
    backward_scheme_kwargs: dict = field(default_factory=dict)
    # not in the reference: RMSNorm and the SwiGLU product are computed inside the activation quantizer of the linear
    # they feed (quartet_amd.fused) instead of being written out; False runs the reference's op-by-op composition
    fuse_producers: bool = True
    # not in the reference (which leaves the choice to torch's dispatcher): which library kernel serves
    # F.scaled_dot_product_attention.  "auto": on a GPU, the memory-efficient kernels first, then flash, then math --
    # on MI355X with this PyTorch the memory-efficient pair runs a causal 16 x 12 x 2048 x 128 bf16 layer, forward and
    # backward, in 2.1 ms against the 3.7 ms of the flash pair the dispatcher picks; "default": the dispatcher's order
    sdpa_backend: str = "auto"

    @property
    def ffn_dim(self):
        """2/3 of 4d, rounded up to ``multiple_of`` (llama.py:82-88)."""
        hidden = int(2 * (4 * self.n_embd) / 3)
        return self.multiple_of * ((hidden + self.multiple_of - 1) // self.multiple_of)


def llama_30m(**overrides):
    """30 M-parameter configuration: 6 layers, d 640, 5 heads, SwiGLU width 1728 (multiple_of 64)."""
    return LlamaConfig(**{**dict(n_layer=6, n_head=5, n_embd=640, multiple_of=64, sequence_length=512), **overrides})


def llama_800m(**overrides):
    """~800 M-parameter configuration: 24 layers, d 1536, 12 heads, SwiGLU width 4096, sequence 2048."""
    return LlamaConfig(**{**dict(n_layer=24, n_head=12, n_embd=1536, multiple_of=256, sequence_length=2048), **overrides})


def unquantized(**overrides):
    """Overrides selecting the bf16 baseline: identity quantizers and the plain scheme."""
    return {**dict(w_quant="NoQuantizer", w_quant_kwargs={}, a_quant="NoQuantizer", a_quant_kwargs={},
                   g_quant="NoQuantizer", g_quant_kwargs={}, backward_scheme="EW_EtX", backward_scheme_kwargs={}),
            **overrides}


def _linear(config, fan_in, fan_out):
    return QuantizedLinear(
        fan_in, fan_out, bias=config.bias,
        weight_quantizer=QUANTIZER_CLASSES[config.w_quant](**config.w_quant_kwargs),
        activation_quantizer=QUANTIZER_CLASSES[config.a_quant](**config.a_quant_kwargs),
        gradient_quantizer=QUANTIZER_CLASSES[config.g_quant](**config.g_quant_kwargs),
        backward_scheme=BACKWARD_SCHEMES[config.backward_scheme](**config.backward_scheme_kwargs),
    )


def rotary_table(head_dim, length, theta=10000.0):
    """[length, head_dim/2, 2] fp32 table of (cos, sin) of position * theta^(-2i/head_dim) (llama.py:17-25)."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2)[: head_dim // 2].float() / head_dim))
    ang = torch.outer(torch.arange(length), inv).float()
    return torch.stack((torch.cos(ang), torch.sin(ang)), dim=-1)


def apply_rotary(q, k, table):
    """Rotate consecutive element pairs (2i, 2i+1) of q, k [B, T, heads, head_dim] by the table's angles, in
    fp32; returns fp32 tensors (llama.py:43-61)."""
    cos, sin = table[:, None, :, 0], table[:, None, :, 1]  # [T, 1, head_dim/2]

    def rot(t):
        pairs = t.float().unflatten(-1, (-1, 2))
        a, b = pairs[..., 0], pairs[..., 1]
        return torch.stack((a * cos - b * sin, a * sin + b * cos), dim=-1).flatten(-2)
    return rot(q), rot(k)


class RMSNorm(nn.Module):
    """x * rsqrt(mean(x^2) + eps) in fp32, cast back, then the learned gain (llama.py:64-75)."""

    def __init__(self, dim, eps=1e-6):
        super().__init__()
        self.eps = eps
        self.weight = nn.Parameter(torch.ones(dim))

    def forward(self, x):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)).type_as(x) * self.weight


class LlamaMLP(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.hidden_dim = config.ffn_dim
        self.w12 = _linear(config, config.n_embd, 2 * self.hidden_dim)
        self.c_proj = _linear(config, self.hidden_dim, config.n_embd)

    def forward(self, x, norm=None, add=None):
        """`norm`: the block's RMSNorm, applied to x (+ `add`, the attention branch's output) here, fused into w12's
        quantizer, instead of by the caller."""
        if norm is not None:   # returns (mlp output, x + add for the residual sum)
            h12, x = rmsnorm_linear(norm, self.w12, x, pass_input=True, add=add)
            return swiglu_linear(self.c_proj, h12), x
        up, gate = self.w12(x).split(self.hidden_dim, dim=-1)
        return self.c_proj(F.silu(up) * gate)


def _sdpa_choice(mode, q):
    """Context manager that sets the order in which scaled_dot_product_attention tries its library kernels."""
    if mode not in ("auto", "default"):
        raise ValueError(f"sdpa_backend must be 'auto' or 'default', got {mode!r}")
    if mode == "default" or not q.is_cuda:
        return contextlib.nullcontext()
    return sdpa_kernel([SDPBackend.EFFICIENT_ATTENTION, SDPBackend.FLASH_ATTENTION, SDPBackend.MATH], set_priority=True)


class LlamaAttention(nn.Module):
    def __init__(self, config):
        super().__init__()
        assert config.n_embd % config.n_head == 0
        self.c_attn = _linear(config, config.n_embd, 3 * config.n_embd)
        self.c_proj = _linear(config, config.n_embd, config.n_embd)
        self.resid_dropout = nn.Dropout(config.dropout)
        self.n_head, self.n_embd, self.dropout = config.n_head, config.n_embd, config.dropout
        self.sdpa_backend = config.sdpa_backend

    def forward(self, x, table, norm=None, add=None):
        B, T, C = x.shape
        hs = C // self.n_head
        if norm is None:
            qkv = self.c_attn(x)
        else:
            qkv, x = rmsnorm_linear(norm, self.c_attn, x, pass_input=True, add=add)
        if norm is not None:   # the fused path: split, rotate and convert in one kernel
            q, k, v = rope_qkv(qkv, table, self.n_head)
        else:
            q, k, v = qkv.split(self.n_embd, dim=2)
            q, k = apply_rotary(q.view(B, T, self.n_head, hs), k.view(B, T, self.n_head, hs), table)
            v = v.view(B, T, self.n_head, hs)
        q, k, v = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
        if not torch.is_autocast_enabled() and v.dtype != q.dtype:
            v = v.to(q.dtype)
        with _sdpa_choice(self.sdpa_backend, q):
            y = F.scaled_dot_product_attention(q, k, v, attn_mask=None, dropout_p=self.dropout, is_causal=True)
        y = y.transpose(1, 2).contiguous().view(B, T, C)
        out = self.resid_dropout(self.c_proj(y))
        return out if norm is None else (out, x)   # with the fused norm: also x for the residual sum


class LlamaBlock(nn.Module):
    def __init__(self, config):
        super().__init__()
        self.ln_1 = RMSNorm(config.n_embd, eps=config.rmsnorm_eps)
        self.attn = LlamaAttention(config)
        self.ln_2 = RMSNorm(config.n_embd, eps=config.rmsnorm_eps)
        self.mlp = LlamaMLP(config)
        self.fuse_producers = config.fuse_producers

    def forward(self, x, table, pending=None):
        """Fused form: returns (x, m) with the block's output x + m left to whoever consumes it -- the next block's first
        norm forms it inside its quantizer kernel (`pending`), as this block's second norm does with x + attention."""
        if self.fuse_producers:
            a, x = self.attn(x, table, norm=self.ln_1, add=pending)
            return self.mlp(x, norm=self.ln_2, add=a)[::-1]
        x = x + self.attn(self.ln_1(x), table)
        return x + self.mlp(self.ln_2(x))


class Llama(nn.Module):
    """Token ids [B, S] -> {"logits", "loss"} (llama.py:177-262)."""

    def __init__(self, config):
        super().__init__()
        self.config = config
        self.head_dim = config.n_embd // config.n_head
        self.register_buffer("freqs_cis", rotary_table(self.head_dim, config.sequence_length), persistent=False)
        self.transformer = nn.ModuleDict(dict(
            wte=nn.Embedding(config.vocab_size, config.n_embd),
            drop=nn.Dropout(config.dropout),
            h=nn.ModuleList([LlamaBlock(config) for _ in range(config.n_layer)]),
            ln_f=RMSNorm(config.n_embd, eps=config.rmsnorm_eps),
        ))
        self.lm_head = nn.Linear(config.n_embd, config.vocab_size, bias=False)
        self.apply(self._init_weights)
        for name, p in self.named_parameters():
            if name.endswith("c_proj.weight"):
                nn.init.normal_(p, mean=0.0, std=config.init_std / math.sqrt(2 * config.n_layer))

    def _init_weights(self, module):
        # QuantizedLinear is an nn.Linear, so the block linears are initialised here too (base.py:229-235)
        if isinstance(module, nn.Linear):
            nn.init.normal_(module.weight, mean=0.0, std=self.config.init_std)
            if module.bias is not None:
                nn.init.zeros_(module.bias)
        elif isinstance(module, nn.Embedding):
            nn.init.normal_(module.weight, mean=0.0, std=self.config.init_std)

    def get_num_params(self, non_embedding=True):
        return sum(p.numel() for p in self.parameters())

    def block_linears(self):
        """(name, module) of every quantized linear, in forward order."""
        return [(n, m) for n, m in self.named_modules() if isinstance(m, QuantizedLinear)]

    def forward(self, idx, targets=None, get_logits=False):
        b, t = idx.shape
        assert t <= self.config.sequence_length, f"sequence of length {t} exceeds block size {self.config.sequence_length}"
        x = self.transformer.drop(self.transformer.wte(idx))
        table = self.freqs_cis[:t]
        pending = None   # a block's MLP output, not yet added to the residual stream (fused blocks only)
        for block in self.transformer.h:
            if block.fuse_producers:
                x, pending = block(x, table, pending)
            else:
                x = block(x if pending is None else x + pending, table)
                pending = None
        if pending is not None:
            x = x + pending
        x = self.transformer.ln_f(x)
        if targets is not None:
            logits = self.lm_head(x)
            loss = F.cross_entropy(logits.view(-1, logits.size(-1)), targets.view(-1), ignore_index=-1)
        else:
            logits = self.lm_head(x[:, [-1], :])
            loss = None
        return {"logits": logits if get_logits else None, "loss": loss}
