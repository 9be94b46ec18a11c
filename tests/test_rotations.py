"""CPU tests of the quantizer modules' rotation state: accumulated sign flips, the dense random rotation of
rerotate="O32", the classifier that tells the two apart, and the oracle's pass-through mode for rotated input."""
import numpy as np
import pytest
import torch

import quartet_amd as q
from quartet_amd.quantizers.mxfp4 import sylvester_matrix, sylvester_sign_bits
from tests.util import make_input, to_oracle


@pytest.mark.parametrize("cls", [q.QuestMXFP4Quantizer, q.AlbertTsengQuantizer, q.AlignedAlbertTsengQuantizer])
@pytest.mark.parametrize("hd", [32, 64])
def test_o32_gives_a_fresh_orthogonal_matrix(cls, hd):
    torch.manual_seed(hd)
    quant = cls(hadamard_dim=hd, rerotate="O32")
    assert not quant.is_dense and sylvester_sign_bits(quant.hadamard_matrix) == 0
    quant.re_randomize()
    r1 = quant.hadamard_matrix
    assert quant.is_dense and r1.shape == (hd, hd) and r1.dtype == torch.float32
    assert torch.allclose(r1.T @ r1, torch.eye(hd), atol=1e-5)
    assert sylvester_sign_bits(r1) is None
    quant.re_randomize()
    assert not torch.equal(quant.hadamard_matrix, r1)
    quant._note_input(torch.zeros(1, dtype=torch.bfloat16))
    assert quant.hadamard_matrix.dtype == torch.bfloat16


def test_sign_flips_accumulate_and_other_values_are_checked():
    torch.manual_seed(3)
    quant = q.AlbertTsengQuantizer(rerotate="signs")
    h = quant.hadamard_matrix
    for _ in range(4):
        flips = None
        state = torch.get_rng_state()
        quant.re_randomize()
        torch.set_rng_state(state)
        flips = torch.randint(0, 2, (32,)) * 2.0 - 1.0          # the draw re_randomize just made
        h = h @ torch.diag(flips)
        assert torch.equal(quant.hadamard_matrix, h)
        assert sylvester_sign_bits(quant.hadamard_matrix) == quant.sign_bits
    fixed = q.QuestMXFP4Quantizer(rerotate=None)
    fixed.re_randomize()
    assert fixed.sign_bits == 0 and not fixed.is_dense
    with pytest.raises(ValueError):
        q.AlbertTsengQuantizer(rerotate="haar").re_randomize()
    with pytest.raises(ValueError):
        q.QuestMXFP4Quantizer(hadamard_dim=16)


def test_classifier_tells_signed_sylvester_from_everything_else():
    h = sylvester_matrix(32) * torch.tensor(32 ** -0.5)
    assert sylvester_sign_bits(h) == 0 and sylvester_sign_bits(h.to(torch.bfloat16)) == 0
    assert sylvester_sign_bits(-h) == 2 ** 32 - 1
    assert sylvester_sign_bits(h * 2) is None and sylvester_sign_bits(h[:, :16]) is None
    assert sylvester_sign_bits(torch.eye(32)) is None and sylvester_sign_bits(torch.eye(16)) is None
    assert sylvester_sign_bits(torch.linalg.qr(torch.randn(32, 32))[0]) is None


def test_layer_with_a_dense_rotation_takes_the_generic_path():
    make = lambda rr: q.QuantizedLinear(64, 64, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
                                        activation_quantizer=q.QuestMXFP4Quantizer(),
                                        gradient_quantizer=q.AlbertTsengQuantizer(stochastic=True, rerotate=rr),
                                        backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]())
    assert make("signs")._is_production_config()
    assert not make("O32")._is_production_config()


@pytest.mark.parametrize("mode", ["QUEST_RTN", "ABSMAX_RTN", "ABSMAX_SR"])
def test_oracle_pass_through_mode_equals_quantizing_its_own_rotated_tensor(oracle, mode):
    """Block size 1 = "already rotated": feeding the fp32 rotated tensor the block-32 run reports must reproduce
    that run's codes, scales and mask (same group values, same Philox offsets)."""
    x = make_input(24, 256, torch.bfloat16, seed=8)
    signs = np.where(np.arange(32) % 3 == 0, -1.0, 1.0)
    m = getattr(oracle, mode)
    full = oracle.quantize(to_oracle(x), 32, signs=signs, mode=m, seed=99, want_mask=True, want_rotated=True, want_dequant=True)
    again = oracle.quantize(full["rotated"], 1, mode=m, seed=99, want_mask=True, want_dequant=True)
    for key in ("codes", "scales", "mask"):
        assert np.array_equal(full[key], again[key]), key
    # the de-quantized values agree once the fp32 ones are rounded to the block-32 run's bf16
    back = torch.from_numpy(again["dequant"]).to(torch.bfloat16)
    assert np.array_equal(to_oracle(back), full["dequant"])
    with pytest.raises(ValueError):
        oracle.quantize(np.zeros((4, 48), dtype=np.float32), 1)   # groups of 32 still need cols % 32 == 0
