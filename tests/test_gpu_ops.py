"""GPU tests of the ``quartet::`` operators: each operator against the oracle, and the operator chain
(``PackedLinearFn``) against the fused whole-layer entry points, bit for bit under the same seeds."""
import random

import numpy as np
import pytest
import torch

from tests.util import make_input, to_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import quartet_amd.ops as o
    return o


def rotation(hd, signs, dtype):
    from quartet_amd.quantizers.mxfp4 import sylvester_matrix
    return (sylvester_matrix(hd) * torch.tensor(hd ** -0.5) * signs[None, :]).to(dtype).to(DEV)


def random_signs(hd, seed):
    return torch.randint(0, 2, (hd,), generator=torch.Generator().manual_seed(seed)) * 2.0 - 1.0


@pytest.mark.parametrize("hd", [32, 64, 128])
def test_quest_operator_against_oracle(oracle, ops, hd):
    print(f"case fusedQuantizeMx_op hd={hd}", flush=True)
    signs = random_signs(hd, hd)
    x = make_input(96, 512, torch.bfloat16, seed=3)
    c, s, m = ops.fusedQuantizeMx_op(x.to(DEV), rotation(hd, signs, torch.bfloat16), True)
    want = oracle.quantize(to_oracle(x), hd, signs=signs.numpy(), mode=oracle.QUEST_RTN, want_mask=True)
    assert np.array_equal(to_oracle(c), want["codes"])
    assert np.array_equal(to_oracle(s), want["scales"])
    assert np.array_equal(to_oracle(m), want["mask"])
    c2, s2, none = ops.fusedQuantizeMx_op(x.to(DEV), rotation(hd, signs, torch.bfloat16), False)
    assert none.numel() == 0 and torch.equal(c2, c) and torch.equal(s2, s)


def test_gradient_side_operators_against_oracle(oracle, ops):
    print("case absmax / transposed / requantize operators", flush=True)
    signs = random_signs(32, 11)
    h = rotation(32, signs, torch.bfloat16)
    g = make_input(128, 192, torch.bfloat16, seed=4, scale=1e-3)
    random.seed(77)
    seeds = [random.getrandbits(63) for _ in range(3)]
    random.seed(77)
    c, s = ops.fusedQuantizeMxAbsMax_op(g.to(DEV), h, True)
    ct, st = ops.backward_t_bf16_op(g.to(DEV), h)
    quarter = torch.full((1,), 0.25, device=DEV)
    cq, sq = ops.backward_qt_bf16_op(c, s, h, quarter)
    w1 = oracle.quantize(to_oracle(g), 32, signs=signs.numpy(), mode=oracle.ABSMAX_SR, seed=seeds[0])
    w2 = oracle.quantize(to_oracle(g), 32, signs=signs.numpy(), mode=oracle.ABSMAX_SR, transposed_in=True, seed=seeds[1])
    w3 = oracle.requantize_transposed(w1["codes"], w1["scales"], post=0.25, val_dtype=oracle.BF16, hd=32, signs=signs.numpy(),
                                      mode=oracle.ABSMAX_SR, seed=seeds[2])
    for got, want in ((c, w1["codes"]), (s, w1["scales"]), (ct, w2["codes"]), (st, w2["scales"]), (cq, w3["codes"]),
                      (sq, w3["scales"])):
        assert np.array_equal(to_oracle(got), want)
    # round-to-nearest variant draws no seed
    state = random.getstate()
    c0, s0 = ops.fusedQuantizeMxAbsMax_op(g.to(DEV), h, False)
    assert random.getstate() == state
    w0 = oracle.quantize(to_oracle(g), 32, signs=signs.numpy(), mode=oracle.ABSMAX_RTN)
    assert np.array_equal(to_oracle(c0), w0["codes"]) and np.array_equal(to_oracle(s0), w0["scales"])


def test_matmul_and_inverse_rotation_operators(oracle, ops):
    print("case matmul_mxf4_bf16_tn_op / maskedHadamardBwd_op", flush=True)
    from quartet_amd import kernels as K
    h = rotation(32, torch.ones(32), torch.bfloat16)
    a = make_input(192, 256, torch.bfloat16, seed=5)
    b = make_input(320, 256, torch.bfloat16, seed=6, scale=0.02)
    ac, as_, am = ops.fusedQuantizeMx_op(a.to(DEV), h, True)
    bc, bs, _ = ops.fusedQuantizeMx_op(b.to(DEV), h, False)
    alpha = torch.full((1,), 0.375, device=DEV)
    y = ops.matmul_mxf4_bf16_tn_op(ac, bc, as_, bs, alpha)
    assert y.dtype == torch.bfloat16 and y.shape == (192, 320)
    want = 0.375 * oracle.gemm_tn(to_oracle(ac), to_oracle(as_), to_oracle(bc), to_oracle(bs))
    err = np.linalg.norm(y.float().cpu().numpy() - want) / np.linalg.norm(want)
    assert err <= 3e-3  # bf16 output rounding (2^-9 per element) on top of the 1e-3 accumulation bound
    assert torch.equal(y, K.gemm_mxfp4_tn(ac, as_, bc, bs, 0.375, torch.bfloat16))
    # a float8_e8m0fnu view of the scales is accepted, as the reference passes them
    y8 = ops.matmul_mxf4_bf16_tn_op(ac, bc, as_.view(torch.float8_e8m0fnu), bs.view(torch.float8_e8m0fnu), alpha)
    assert torch.equal(y8, y)
    alpha.mul_(2)  # an in-place update of alpha must be seen
    assert torch.equal(ops.matmul_mxf4_bf16_tn_op(ac, bc, as_, bs, alpha).float(), 2 * y.float())
    g = make_input(192, 256, torch.bfloat16, seed=7).to(DEV)
    signs = random_signs(32, 9)
    hs = rotation(32, signs, torch.bfloat16)
    got = ops.maskedHadamardBwd_op(g, am, hs)
    bits = ((am[..., None] >> torch.arange(8, device=DEV, dtype=torch.uint8)) & 1).view(192, 256).float()
    ref = ((g.float() * bits).view(-1, 32) @ hs.float().T).view(192, 256)
    assert torch.allclose(got.float(), ref, rtol=2 ** -7, atol=1e-6)
    no_mask = ops.maskedHadamardBwd_op(g, torch.empty(0, dtype=torch.uint8, device=DEV), hs)
    assert torch.allclose(no_mask.float(), (g.float().view(-1, 32) @ hs.float().T).view(192, 256), rtol=2 ** -7, atol=1e-6)


def test_dense_rotation_is_rejected(ops):
    q, _ = torch.linalg.qr(torch.randn(32, 32))
    with pytest.raises(ValueError):
        ops.fusedQuantizeMx_op(torch.zeros(32, 64, device=DEV, dtype=torch.bfloat16), q.to(DEV, torch.bfloat16), True)


@pytest.mark.parametrize("T,I,O", [(96, 64, 160), (512, 256, 384)])
def test_operator_chain_equals_fused_layer(ops, T, I, O):
    """PackedLinearFn (eleven operator calls) and QuantizedLinear's production path (two foreign calls) must give
    identical bits: same kernels, same seeds in the same order.  The second shape takes the tiled code layout in
    the fused path and row-major codes in the operator chain."""
    print(f"case operator chain vs fused layer T={T} I={I} O={O}", flush=True)
    import quartet_amd as q
    x = make_input(T, I, torch.bfloat16, seed=21, outlier_frac=0.01).to(DEV)
    w = (0.02 * make_input(O, I, torch.bfloat16, seed=22, outlier_frac=0).float()).to(torch.bfloat16).to(DEV)
    dy = make_input(T, O, torch.bfloat16, seed=23, scale=1e-3).to(DEV)
    layer = q.QuantizedLinear(I, O, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
                              activation_quantizer=q.QuestMXFP4Quantizer(),
                              gradient_quantizer=q.AlbertTsengQuantizer(stochastic=True, rerotate="signs"),
                              backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(DEV, torch.bfloat16)
    with torch.no_grad():
        layer.weight.copy_(w)
    xa = x.clone().requires_grad_(True)
    torch.manual_seed(3)
    random.seed(5)
    ya = layer(xa)
    ya.backward(dy)
    g_q = layer.backward_scheme.g_quantizer

    xb = x.clone().requires_grad_(True)
    wb = w.clone().requires_grad_(True)
    hf = layer.activation_quantizer.hadamard_matrix.to(DEV, torch.bfloat16)
    hb = g_q.hadamard_matrix.to(DEV, torch.bfloat16)  # the signs the fused backward used
    random.seed(5)
    yb = ops.PackedLinearFn.apply(xb, wb, hf, hb)
    yb.backward(dy)
    assert torch.equal(ya, yb)
    assert torch.equal(xa.grad, xb.grad)
    assert torch.equal(layer.weight.grad, wb.grad)


def test_operator_chain_compiles_fullgraph(ops):
    """torch.compile(fullgraph=True) traces through the operators by their shape functions (the reason the reference
    registers them); the compiled forward must reproduce the eager result."""
    print("case torch.compile fullgraph over the operator chain", flush=True)
    h = rotation(32, torch.ones(32), torch.bfloat16)
    x = make_input(128, 256, torch.bfloat16, seed=31).to(DEV)
    w = make_input(192, 256, torch.bfloat16, seed=32, scale=0.02).to(DEV)

    def fwd(x, w, h):
        return ops.packed_forward(x, w, h)[0]
    eager = fwd(x, w, h)
    compiled = torch.compile(fwd, fullgraph=True, backend="aot_eager")
    assert torch.equal(compiled(x, w, h), eager)
    assert torch.equal(compiled(x, w, h), eager)
