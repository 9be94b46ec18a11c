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


def test_device_seed_base_shifts_every_seed():
    """qm_linear_backward_seeded with the value v behind seed_base == qm_linear_backward with seeds + v, bit for bit."""
    from quartet_amd import kernels as K
    dev = torch.device("cuda:0")
    T, I, O = 512, 384, 640
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, I, generator=g).bfloat16().to(dev)
    w = (0.02 * torch.randn(O, I, generator=g)).to(dev)
    e = (1e-3 * torch.randn(T, O, generator=g)).bfloat16().to(dev)
    _, px, pw = K.linear_forward(x, w, 32, None, 32, None, torch.bfloat16, True)
    seeds, signs_g, v = (21, 22, 23, 24), 0x0F0F3C3C, 1000003

    def backward(sd, base):
        return K.linear_backward(e, px, pw, T, I, O, 32, None, 32, None, 32, signs_g, K.QM_ABSMAX_SR, sd, x.dtype, w.dtype,
                                 torch.bfloat16, torch.bfloat16, torch.bfloat16, True, False, torch.float32, None, base)
    base = torch.tensor([v], dtype=torch.int64, device=dev)
    shifted = backward(seeds, base)
    direct = backward(tuple(s + v for s in seeds), None)
    unshifted = backward(seeds, None)
    for a, b in zip(shifted, direct):
        assert torch.equal(a, b)
    assert not torch.equal(shifted[0], unshifted[0]) and not torch.equal(shifted[1], unshifted[1])
    # a zero base is the plain call
    base.zero_()
    for a, b in zip(backward(seeds, base), unshifted):
        assert torch.equal(a, b)
    # shapes off the tiled layout refuse a seed base instead of ignoring it
    from quartet_amd import _lib
    with pytest.raises(_lib.QuartetHipError):
        K.linear_backward(e[:, :32].contiguous(), px, pw, T, I, 32, 32, None, 32, None, 32, signs_g, K.QM_ABSMAX_SR, seeds, x.dtype,
                          w.dtype, torch.bfloat16, torch.bfloat16, torch.bfloat16, False, False, torch.float32, None, base)


def test_captured_layer_step_draws_fresh_streams_with_a_seed_base():
    """A QuantizedLinear step captured once: with a device seed base that the graph increments, every replay rounds the
    gradients with new random streams; replay k equals the eager kernels with the capture's seeds shifted by k."""
    import quartet_amd as q
    from quartet_amd import kernels as K
    from quartet_amd.quantizers import mxfp4
    dev = torch.device("cuda:0")
    T, I, O = 512, 256, 384
    layer = q.QuantizedLinear(
        I, O, bias=False,
        weight_quantizer=q.QUANTIZER_CLASSES["QuestMXFP4Quantizer"](hadamard_dim=32),
        activation_quantizer=q.QUANTIZER_CLASSES["QuestMXFP4Quantizer"](hadamard_dim=32),
        gradient_quantizer=q.QUANTIZER_CLASSES["AlbertTsengQuantizer"](hadamard_dim=32, stochastic=True, rerotate="signs"),
        backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(device=dev, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(T, I, generator=g).bfloat16().to(dev).requires_grad_(True)
    e = (1e-3 * torch.randn(T, O, generator=g)).bfloat16().to(dev)
    base = torch.zeros(1, dtype=torch.int64, device=dev)
    drawn = []
    real_seed = mxfp4._fresh_seed

    def recording_seed():
        drawn.append(real_seed())
        return drawn[-1]
    import quartet_amd.linear as lin
    old = lin._fresh_seed
    lin._fresh_seed = recording_seed
    q.set_device_seed_base(base)
    try:
        def step():
            y = layer(x)
            return torch.autograd.grad(y, (x, layer.weight), e)
        step()                                    # warm-up outside the capture
        torch.cuda.synchronize()
        drawn.clear()
        base.zero_()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            gx_g, gw_g = step()
            base.add_(1)
        seeds = tuple(drawn[-4:])
        signs_g = layer.backward_scheme.g_quantizer.sign_bits
        _, px, pw = K.linear_forward(x.detach(), layer.weight.detach(), 32, None, 32, None, torch.bfloat16, True)
        base.zero_()
        seen = []
        for k in range(3):
            graph.replay()
            torch.cuda.synchronize()
            assert int(base.item()) == k + 1
            want = K.linear_backward(e, px, pw, T, I, O, 32, None, 32, None, 32, signs_g, K.QM_ABSMAX_SR,
                                     tuple(s + k for s in seeds), torch.bfloat16, torch.bfloat16, torch.bfloat16, torch.bfloat16,
                                     torch.bfloat16, True, False, torch.bfloat16)
            assert torch.equal(gx_g, want[0]) and torch.equal(gw_g, want[1]), f"replay {k}"
            seen.append(gx_g.clone())
        assert not torch.equal(seen[0], seen[1]) and not torch.equal(seen[1], seen[2])
    finally:
        lin._fresh_seed = old
        q.set_device_seed_base(None)


def test_seed_base_refuses_layers_that_would_ignore_it():
    """With a device seed base set, a stochastic layer whose shape keeps it off the tiled layout must fail loudly: its
    kernels take host seeds only, so a captured replay would repeat their random streams."""
    import quartet_amd as q
    from quartet_amd import _lib
    dev = torch.device("cuda:0")
    layer = q.QuantizedLinear(96, 160, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(), activation_quantizer=q.QuestMXFP4Quantizer(),
                              gradient_quantizer=q.AlbertTsengQuantizer(stochastic=True, rerotate="signs"),
                              backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(dev, torch.bfloat16)
    x = torch.randn(64, 96, device=dev, dtype=torch.bfloat16, requires_grad=True)
    q.set_device_seed_base(torch.zeros(1, dtype=torch.int64, device=dev))
    try:
        with pytest.raises(_lib.QuartetHipError, match="seed base"):
            layer(x).sum().backward()
    finally:
        q.set_device_seed_base(None)
    layer(x).sum().backward()      # without a seed base the same layer runs
    assert torch.isfinite(x.grad.float()).all()


def test_sign_flips_of_the_gradient_rotation_cancel_in_both_products():
    """Why a captured step needs no device-side sign words: the gradient quantizer's sign flips (re_randomize("signs"),
    mxfp4.py:53-60) multiply both operands of each backward product along the contracted index, and the absmax
    quantizers are odd, so gx and gw do not depend on them, bit for bit."""
    from quartet_amd import kernels as K
    dev = torch.device("cuda:0")
    T, I, O = 512, 384, 640
    g = torch.Generator().manual_seed(6)
    x = torch.randn(T, I, generator=g).bfloat16().to(dev)
    w = (0.02 * torch.randn(O, I, generator=g)).to(dev)
    e = (1e-3 * torch.randn(T, O, generator=g)).bfloat16().to(dev)
    _, px, pw = K.linear_forward(x, w, 32, None, 32, None, torch.bfloat16, True)
    for mode in (K.QM_ABSMAX_SR, K.QM_ABSMAX_RTN):
        outs = [K.linear_backward(e, px, pw, T, I, O, 32, None, 32, None, 32, sg, mode, (31, 32, 33, 34), x.dtype, w.dtype,
                                  torch.bfloat16, torch.bfloat16, torch.bfloat16, True, False, torch.float32)
                for sg in (0, 0x0F0F3C3C, 0xFFFFFFFF, 0x80000001)]
        for o in outs[1:]:
            assert torch.equal(o[0], outs[0][0]) and torch.equal(o[1], outs[0][1])
