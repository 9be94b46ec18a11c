"""The Llama caller model (quartet_amd/llama.py) against what fixes it without running the reference:
closed-form parameter counts of the two published configurations, loss at initialisation on uniform ids,
bit-equality of the identity-quantizer configuration with a stock nn.Linear model, and textbook properties
of the rotary embedding and RMSNorm.  CPU only."""
import copy
import math

import pytest
import torch
import torch.nn as nn

from quartet_amd import llama as L
from quartet_amd.linear import QuantizedLinear


def test_ffn_width_rule():
    assert L.llama_30m().ffn_dim == 1728          # int(2*2560/3) = 1706 -> next multiple of 64
    assert L.LlamaConfig(n_embd=640).ffn_dim == 1792  # the default multiple_of = 256
    assert L.llama_800m().ffn_dim == 4096


@pytest.mark.parametrize("make,per_layer,embed", [
    (L.llama_30m, 640 * 1920 + 640 * 640 + 640 * 3456 + 1728 * 640, 32000 * 640),
    (L.llama_800m, 1536 * 4608 + 1536 * 1536 + 1536 * 8192 + 4096 * 1536, 32000 * 1536),
])
def test_parameter_counts_closed_form(make, per_layer, embed):
    cfg = make(**L.unquantized())
    with torch.device("meta"):
        m = L.Llama(cfg)
    lin = sum(mod.weight.numel() for _, mod in m.block_linears())
    assert lin == per_layer * cfg.n_layer
    assert len(m.block_linears()) == 4 * cfg.n_layer
    norms = (2 * cfg.n_layer + 1) * cfg.n_embd
    assert m.get_num_params() == lin + 2 * embed + norms
    if make is L.llama_30m:
        assert lin == 29_736_960
    else:
        assert lin == 679_477_248
    # fused projections: c_attn is d -> 3d, w12 is d -> 2 d_ff, and no block linear has a bias
    blk = m.transformer.h[0]
    assert blk.attn.c_attn.weight.shape == (3 * cfg.n_embd, cfg.n_embd)
    assert blk.mlp.w12.weight.shape == (2 * cfg.ffn_dim, cfg.n_embd)
    assert all(mod.bias is None for _, mod in m.block_linears())
    assert m.lm_head.weight is not m.transformer.wte.weight  # untied


def _tiny(**kw):
    return L.LlamaConfig(**{**dict(vocab_size=32000, sequence_length=64, n_layer=2, n_head=2, n_embd=128, multiple_of=64),
                            **L.unquantized(), **kw})


def test_loss_at_init_is_log_vocab():
    torch.manual_seed(0)
    m = L.Llama(_tiny())
    idx = torch.randint(0, 32000, (4, 64))
    tgt = torch.randint(0, 32000, (4, 64))
    out = m(idx, targets=tgt)
    assert out["logits"] is None
    # logits are ~N(0, d * init_std^2) and independent of the targets: E[loss] = ln V + d * init_std^2 / 2
    assert abs(float(out["loss"].detach()) - (math.log(32000) + 128 * 0.02 ** 2 / 2)) < 0.1
    last = m(idx, get_logits=True)
    assert last["loss"] is None and last["logits"].shape == (4, 1, 32000)


def test_init_scales():
    torch.manual_seed(1)
    cfg = _tiny(n_layer=3, n_embd=256, n_head=4)
    m = L.Llama(cfg)
    blk = m.transformer.h[0]
    for w, std in ((blk.attn.c_attn.weight, 0.02), (blk.mlp.w12.weight, 0.02), (m.lm_head.weight, 0.02),
                   (m.transformer.wte.weight, 0.02), (blk.attn.c_proj.weight, 0.02 / math.sqrt(6)),
                   (blk.mlp.c_proj.weight, 0.02 / math.sqrt(6))):
        assert abs(float(w.std()) / std - 1.0) < 0.03
    assert torch.equal(blk.ln_1.weight, torch.ones(256))


def test_identity_quantizers_equal_stock_linear_model_bit_for_bit():
    torch.manual_seed(2)
    m = L.Llama(_tiny())
    twin = copy.deepcopy(m)
    for name, mod in list(twin.named_modules()):
        for child_name, child in list(mod.named_children()):
            if isinstance(child, QuantizedLinear):
                plain = nn.Linear(child.in_features, child.out_features, bias=False)
                plain.weight = child.weight
                setattr(mod, child_name, plain)
    assert not any(isinstance(x, QuantizedLinear) for x in twin.modules())
    idx = torch.randint(0, 32000, (2, 48))
    tgt = torch.randint(0, 32000, (2, 48))
    la = m(idx, targets=tgt)["loss"]
    lb = twin(idx, targets=tgt)["loss"]
    assert torch.equal(la, lb)
    la.backward()
    lb.backward()
    ga = dict(m.named_parameters())
    for n, p in twin.named_parameters():
        assert torch.equal(p.grad, ga[n].grad), n


def test_rotary_matches_complex_multiplication_and_is_relative():
    torch.manual_seed(3)
    B, T, H, D = 2, 16, 3, 8
    q, k = torch.randn(B, T, H, D), torch.randn(B, T, H, D)
    table = L.rotary_table(D, T)
    rq, rk = L.apply_rotary(q, k, table)
    # independent formulation: complex rotation by exp(i * pos * theta^(-2j/D))
    inv = 1.0 / (10000.0 ** (torch.arange(0, D, 2).double() / D))
    ang = torch.outer(torch.arange(T).double(), inv)
    rot = torch.polar(torch.ones_like(ang), ang)[None, :, None, :]
    want = torch.view_as_real(torch.view_as_complex(q.double().reshape(B, T, H, D // 2, 2)) * rot).reshape(B, T, H, D)
    assert torch.allclose(rq.double(), want, atol=1e-5)
    assert torch.equal(rq[:, 0], q[:, 0])  # position 0 is the identity
    assert torch.allclose(rq.norm(dim=-1), q.norm(dim=-1), rtol=1e-5)
    # scores depend on the position difference only: shift both sequences by 3 positions
    q2, k2 = torch.zeros(B, T, H, D), torch.zeros(B, T, H, D)
    q2[:, 3:], k2[:, 3:] = q[:, :-3], k[:, :-3]
    sq, sk = L.apply_rotary(q2, k2, table)
    s1 = torch.einsum("bthd,bshd->bhts", rq[:, :-3], rk[:, :-3])
    s2 = torch.einsum("bthd,bshd->bhts", sq[:, 3:], sk[:, 3:])
    assert torch.allclose(s1, s2, atol=1e-4)


def test_rmsnorm_closed_form_and_fp32_statistics():
    n = L.RMSNorm(4, eps=1e-5)
    x = torch.tensor([[3.0, -4.0, 0.0, 0.0]])
    want = x / math.sqrt(25.0 / 4 + 1e-5)
    assert torch.allclose(n(x), want, rtol=1e-6)
    xb = (torch.randn(8, 4) * 100).to(torch.bfloat16)
    ref = (xb.float() * torch.rsqrt(xb.float().pow(2).mean(-1, keepdim=True) + 1e-5)).to(torch.bfloat16)
    assert torch.equal(n(xb), (ref * n.weight).to(n(xb).dtype))


def test_swiglu_split_order_is_up_then_gate():
    torch.manual_seed(4)
    cfg = _tiny()
    mlp = L.LlamaMLP(cfg)
    x = torch.randn(3, cfg.n_embd)
    w = mlp.w12.weight
    up, gate = x @ w[: cfg.ffn_dim].T, x @ w[cfg.ffn_dim:].T
    want = (torch.nn.functional.silu(up) * gate) @ mlp.c_proj.weight.T
    assert torch.allclose(mlp(x), want, atol=1e-6)


def test_sdpa_backend_choice_is_validated_and_inert_on_cpu():
    import contextlib
    from quartet_amd.llama import _sdpa_choice
    q = torch.zeros(1, 1, 4, 8)
    assert isinstance(_sdpa_choice("auto", q), contextlib.nullcontext)      # CPU tensors: the dispatcher's own order
    assert isinstance(_sdpa_choice("default", q), contextlib.nullcontext)
    with pytest.raises(ValueError):
        _sdpa_choice("flash", q)
