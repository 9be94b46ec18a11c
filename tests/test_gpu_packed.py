"""GPU tests of the packed-tensor container: packing through the kernels, file round trip back onto the GPU,
de-quantization and un-rotation, and the views into the buffer a layer keeps for its backward pass."""
import numpy as np
import pytest
import torch

from tests.util import make_input, to_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def P():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from quartet_amd import packed
    return packed


@pytest.mark.parametrize("tiled", [False, True])
def test_pack_save_load_dequantize(oracle, P, tmp_path, tiled):
    print(f"case packed round trip tiled={tiled}", flush=True)
    x = make_input(64, 256, torch.bfloat16, seed=9)
    signs = 0x00F0_1234
    p = P.pack_quest(x.to(DEV), 32, signs, tiled=tiled)
    e = P.pack_absmax(x.to(DEV), 32, signs, stochastic=True, seed=123, tiled=tiled)
    svec = np.array([-1.0 if (signs >> j) & 1 else 1.0 for j in range(32)], dtype=np.float32)
    want = oracle.quantize(to_oracle(x), 32, signs=svec, mode=oracle.QUEST_RTN, want_mask=True, want_dequant=True)
    want_e = oracle.quantize(to_oracle(x), 32, signs=svec, mode=oracle.ABSMAX_SR, seed=123, want_dequant=True)
    assert np.array_equal(to_oracle(p.to_layout("rowmajor").codes), want["codes"])
    assert np.array_equal(to_oracle(p.scales), want["scales"]) and np.array_equal(to_oracle(p.maskbits), want["mask"])
    path = tmp_path / "t.safetensors"
    P.save_packed(path, {"x": p, "e": e})
    back = P.load_packed(path, device=DEV)
    assert back["x"].layout == ("tiled" if tiled else "rowmajor") and back["x"].codes.is_cuda
    # de-quantized values are exactly the oracle's pseudo-quantized tensor (bf16 holds them exactly)
    assert np.array_equal(to_oracle(back["x"].dequantize(torch.bfloat16)), want["dequant"])
    assert np.array_equal(to_oracle(back["e"].dequantize(torch.bfloat16)), want_e["dequant"])
    # undoing the rotation gives the input back up to quantization error (about 10 % relative for 4-bit values)
    rec = back["x"].reconstruct(torch.float32).cpu()
    clean = make_input(64, 256, torch.bfloat16, seed=9, outlier_frac=0).float()
    rec_clean = P.pack_quest(clean.to(DEV).to(torch.bfloat16), 32, signs).reconstruct(torch.float32).cpu()
    rel = float((rec_clean - clean).norm() / clean.norm())
    assert 0.05 < rel < 0.2, rel
    assert rec.shape == x.shape


@pytest.mark.parametrize("T,I,O", [(64, 96, 160), (256, 256, 384)])
def test_views_into_the_operand_buffers(P, T, I, O):
    print(f"case saved-buffer views T={T} I={I} O={O}", flush=True)
    import quartet_amd as q
    from quartet_amd import kernels as K
    x = make_input(T, I, torch.bfloat16, seed=3).to(DEV)
    w = make_input(O, I, torch.bfloat16, seed=4, scale=0.02).to(DEV)
    a_q, w_q = q.QuestMXFP4Quantizer(), q.QuestMXFP4Quantizer()
    tiled = all(d % 128 == 0 and d >= 256 for d in (T, I, O))
    y, packed_x, packed_w = K.linear_forward(x, w, 32, 0, 32, 0, torch.bfloat16, tiled)
    xp = P.from_operand_buffer(packed_x, T, I, tiled, a_q)
    wp = P.from_operand_buffer(packed_w, O, I, tiled, w_q)
    assert xp.codes.data_ptr() == packed_x.data_ptr()  # views, not copies
    for got, src in ((xp, x), (wp, w)):
        direct = P.pack_quest(src, 32, 0, tiled=tiled)
        assert torch.equal(got.codes, direct.codes) and torch.equal(got.scales, direct.scales)
        assert torch.equal(got.maskbits, direct.maskbits)
    # the layer's output is the product of the two de-quantized operands
    ref = xp.dequantize(torch.float32) @ wp.dequantize(torch.float32).T
    assert float((y.float() - ref).norm() / ref.norm()) < 5e-3


def test_quantized_checkpoint_of_a_model(P, tmp_path):
    """pack_model_weights -> file -> load: every block linear's packed weight, and the product of a packed activation
    with the reloaded packed weight equals the layer's own forward output."""
    print("case packed model checkpoint", flush=True)
    import quartet_amd as q
    from quartet_amd import kernels as K
    from quartet_amd.llama import Llama, LlamaConfig
    torch.manual_seed(0)
    model = Llama(LlamaConfig(vocab_size=128, sequence_length=64, n_layer=2, n_head=2, n_embd=256, multiple_of=128)).to(DEV)
    packed = P.pack_model_weights(model, tiled=True)
    assert len(packed) == 8 and all(k.endswith(".weight") for k in packed)
    P.save_packed(tmp_path / "model.safetensors", packed, {"model": "toy"})
    back = P.load_packed(tmp_path / "model.safetensors", device=DEV)
    name, layer = model.block_linears()[0]
    wp = back[f"{name}.weight"]
    assert wp.layout == "tiled" and (wp.rows, wp.cols) == tuple(layer.weight.shape)
    x = make_input(256, layer.weight.shape[1], torch.bfloat16, seed=5).to(DEV)
    xp = P.pack_quest(x, 32, layer.activation_quantizer.sign_bits, tiled=True)
    y = K.gemm_mxfp4_tn(xp.codes, xp.scales, wp.codes, wp.scales, 1.0, torch.bfloat16, a_tiled=True, b_tiled=True)
    with torch.no_grad(), torch.autocast("cuda", dtype=torch.bfloat16):
        want = layer(x)
    assert torch.equal(y, want)
