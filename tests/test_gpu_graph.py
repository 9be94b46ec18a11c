"""The whole-layer entry points under HIP graph capture: they allocate nothing, synchronize nothing and take every
host-side argument (sign words, seeds) by value, so a captured forward + backward must replay to the bits of the eager
calls -- also after the static inputs changed, and with eager work and synchronizations between the replays."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _layer_step(K, x, w, e, seeds, signs_g):
    T, I = x.shape
    O = w.shape[0]
    y, px, pw = K.linear_forward(x, w, 32, None, 32, None, torch.bfloat16, True)
    gx, gw = K.linear_backward(e, px, pw, T, I, O, 32, None, 32, None, 32, signs_g, K.QM_ABSMAX_SR, seeds, x.dtype, w.dtype,
                               torch.bfloat16, torch.bfloat16, torch.bfloat16, True, False, torch.float32)
    return y, gx, gw


@pytest.mark.parametrize("T,I,O", [(512, 512, 768), (1024, 1024, 512)])
def test_layer_forward_and_backward_replay_bit_exactly(T, I, O):
    from quartet_amd import kernels as K
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(T + I + O)
    draw = lambda: (torch.randn(T, I, generator=g).bfloat16().to(dev), (0.02 * torch.randn(O, I, generator=g)).to(dev),
                    (1e-3 * torch.randn(T, O, generator=g)).bfloat16().to(dev))
    seeds, signs_g = (11, 12, 13, 14), 0x5A5AA5A5
    x_s, w_s, e_s = draw()                       # static inputs of the graph
    _layer_step(K, x_s, w_s, e_s, seeds, signs_g)   # warm-up outside the capture (module load, function attributes)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs_g = _layer_step(K, x_s, w_s, e_s, seeds, signs_g)
    for rep in range(4):
        if rep:                                  # new contents in the same buffers
            for dst, src in zip((x_s, w_s, e_s), draw()):
                dst.copy_(src)
        eager = [t.clone() for t in _layer_step(K, x_s.clone(), w_s.clone(), e_s.clone(), seeds, signs_g)]
        # unrelated eager work and a synchronization between the replays
        K.quantize_mxfp4(torch.randn(256, 256, device=dev).bfloat16(), 32, None, K.QM_QUEST_RTN, want_mask=True)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("y", "gx", "gw"), outs_g, eager):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager call"
