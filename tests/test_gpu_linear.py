"""GPU parity of the whole Quartet linear (QuantizedLinear in its production configuration and the
per-quantizer modules) against the oracle pipeline on identical inputs, seeds and sign flips."""
import random

import numpy as np
import pytest
import torch

from tests.util import make_input, to_oracle

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def q():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import quartet_amd
    return quartet_amd


def rel(a, b):
    a, b = np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


def production_layer(q, I, O, stochastic, rerotate, dtype):
    return q.QuantizedLinear(I, O, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
                             activation_quantizer=q.QuestMXFP4Quantizer(),
                             gradient_quantizer=q.AlbertTsengQuantizer(stochastic=stochastic, rerotate=rerotate),
                             backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to("cuda:0", dtype)


def oracle_step(o, x, w, dy, signs, seeds, mode, val_dtype):
    d = float(o.FOUR_THIRDS)
    qx = o.quantize(to_oracle(x), 32, mode=o.QUEST_RTN, want_mask=True)
    qw = o.quantize(to_oracle(w), 32, mode=o.QUEST_RTN, want_mask=True)
    y = o.gemm_tn(qx["codes"], qx["scales"], qw["codes"], qw["scales"])
    qe = o.quantize(to_oracle(dy), 32, signs=signs, mode=mode, seed=seeds[0])
    qwt = o.requantize_transposed(qw["codes"], qw["scales"], val_dtype=val_dtype, hd=32, signs=signs, mode=mode, seed=seeds[1])
    gxq = o.gemm_tn(qe["codes"], qe["scales"], qwt["codes"], qwt["scales"], a_post=d, b_post=d)
    qet = o.quantize(to_oracle(dy), 32, signs=signs, mode=mode, transposed_in=True, seed=seeds[2])
    qxt = o.requantize_transposed(qx["codes"], qx["scales"], val_dtype=val_dtype, hd=32, signs=signs, mode=mode, seed=seeds[3])
    gwq = o.gemm_tn(qet["codes"], qet["scales"], qxt["codes"], qxt["scales"], a_post=d, b_post=d)
    return y, gxq, gwq, qx["mask"], qw["mask"]


def test_config1_forward_with_outlier_columns(oracle, q):
    # X [4096 x 512] ~ N(0,1) with 4 outlier columns x20, W [2048 x 512] ~ N(0, 0.02), seed 0
    g = torch.Generator().manual_seed(0)
    x = torch.randn(4096, 512, generator=g)
    cols = torch.randperm(512, generator=g)[:4]
    x[:, cols] *= 20
    w = 0.02 * torch.randn(2048, 512, generator=g)
    x, w = x.to(torch.bfloat16), w.to(torch.bfloat16)
    from quartet_amd import kernels as K
    dev = "cuda:0"
    xc, xs, xm, _ = K.quantize_mxfp4(x.to(dev), 32, None, K.QM_QUEST_RTN, want_mask=True)
    wc, ws, wm, _ = K.quantize_mxfp4(w.to(dev), 32, None, K.QM_QUEST_RTN, want_mask=True)
    qx = oracle.quantize(to_oracle(x), 32, mode=oracle.QUEST_RTN, want_mask=True)
    qw = oracle.quantize(to_oracle(w), 32, mode=oracle.QUEST_RTN, want_mask=True)
    for got, want in ((xc, qx["codes"]), (xs, qx["scales"]), (xm, qx["mask"]), (wc, qw["codes"]), (ws, qw["scales"]), (wm, qw["mask"])):
        assert np.array_equal(to_oracle(got), want)
    y = K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.float32)
    y_ref = oracle.gemm_tn(qx["codes"], qx["scales"], qw["codes"], qw["scales"])
    assert rel(y.cpu().numpy(), y_ref) <= 1e-3
    # and through the module (bf16 output = one extra rounding of 2^-9 relative per element)
    layer = production_layer(q, 512, 2048, False, None, torch.bfloat16)
    with torch.no_grad():
        layer.weight.copy_(w.to(dev))
        ym = layer(x.to(dev))
    assert torch.equal(ym.cpu(), y.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("stochastic,rerotate", [(False, None), (True, "signs")])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_production_step_against_oracle(oracle, q, stochastic, rerotate, dtype):
    print(f"case linear step stochastic={stochastic} rerotate={rerotate} dtype={dtype}", flush=True)
    T, I, O = 384, 256, 160
    x = make_input(T, I, dtype, seed=1, outlier_frac=0.01)
    w = make_input(O, I, dtype, seed=2, outlier_frac=0, scale=0.02)
    dy = make_input(T, O, dtype, seed=3, outlier_frac=0, scale=1e-3)
    layer = production_layer(q, I, O, stochastic, rerotate, dtype)
    with torch.no_grad():
        layer.weight.copy_(w.to("cuda:0"))
    xd = x.to("cuda:0").view(2, T // 2, I).requires_grad_(True)  # leading dims are flattened by the layer
    torch.manual_seed(5)
    random.seed(5)
    y = layer(xd)
    y.backward(dy.to("cuda:0").view(2, T // 2, O))
    torch.cuda.synchronize()

    torch.manual_seed(5)
    random.seed(5)
    signs = None
    if rerotate == "signs":
        signs = np.where(torch.randint(0, 2, (32,)).numpy() == 0, -1, 1)
    seeds = [random.getrandbits(63) for _ in range(4)] if stochastic else [0, 0, 0, 0]
    mode = oracle.ABSMAX_SR if stochastic else oracle.ABSMAX_RTN
    vd = oracle.BF16 if dtype == torch.bfloat16 else oracle.F32
    y_ref, gxq, gwq, xm, wm = oracle_step(oracle, x, w, dy, signs, seeds, mode, vd)
    gx_ref = oracle.masked_hadamard_bwd(gxq.astype(np.float32), 32, vd, None, xm, out_dtype=oracle.F32)
    gw_ref = oracle.masked_hadamard_bwd(gwq.astype(np.float32), 32, vd, None, wm, out_dtype=oracle.F32)
    # fp32 end to end: only accumulation order differs -> the 1e-3 Frobenius tolerance of the target,
    # with a wide margin.  bf16: each stored tensor adds one rounding of relative size 2^-9.
    tol_y, tol_g = (1e-5, 1e-5) if dtype == torch.float32 else (3e-3, 5e-3)
    assert y.dtype == dtype and xd.grad.dtype == dtype and layer.weight.grad.dtype == dtype
    assert rel(y.detach().float().cpu().numpy().reshape(T, O), y_ref) <= tol_y
    assert rel(xd.grad.float().cpu().numpy().reshape(T, I), gx_ref) <= tol_g
    assert rel(layer.weight.grad.float().cpu().numpy(), gw_ref) <= tol_g


def test_generic_module_path_matches_packed_path(q):
    # the reference-shaped path (quantizer modules -> de-quantized tensors -> library GEMMs) and the
    # packed FP4 path compute the same function when the backward is deterministic
    T, I, O = 256, 128, 96
    x = make_input(T, I, torch.float32, seed=4)
    w = make_input(O, I, torch.float32, seed=5, outlier_frac=0, scale=0.02)
    dy = make_input(T, O, torch.float32, seed=6, outlier_frac=0, scale=1e-3)
    outs = []
    for packed in (True, False):
        layer = production_layer(q, I, O, False, None, torch.float32)
        layer.use_packed_path = packed
        with torch.no_grad():
            layer.weight.copy_(w.to("cuda:0"))
        xd = x.to("cuda:0").requires_grad_(True)
        y = layer(xd)
        y.backward(dy.to("cuda:0"))
        outs.append((y.detach().cpu().numpy(), xd.grad.cpu().numpy(), layer.weight.grad.cpu().numpy()))
    for a, b in zip(*outs):
        assert rel(a, b) <= 1e-3


def test_quantizer_modules_match_oracle(oracle, q):
    dev = "cuda:0"
    x = make_input(64, 256, torch.bfloat16, seed=7)
    xd = x.to(dev).requires_grad_(True)
    quest = q.QuestMXFP4Quantizer()
    out = quest(xd)
    ref = oracle.quantize(to_oracle(x), 32, mode=oracle.QUEST_RTN, want_mask=True, want_dequant=True)
    assert np.array_equal(to_oracle(out), ref["dequant"])
    g = make_input(64, 256, torch.bfloat16, seed=8, outlier_frac=0)
    out.backward(g.to(dev))
    want = oracle.masked_hadamard_bwd(to_oracle(g), 32, oracle.BF16, None, ref["mask"])
    assert np.array_equal(to_oracle(xd.grad), want)
    # kernel wrapper with the reference's signature, matrix carrying sign flips
    tseng = q.AlbertTsengQuantizer(stochastic=False, rerotate="signs")
    torch.manual_seed(3)
    tseng.re_randomize()
    tseng._note_input(xd)
    deq, clip = q.mxfp4_forward_kernel_wrapper(x.to(dev), tseng.hadamard_matrix, return_clip_mask=True, quest=False)
    signs = np.array([-1 if (tseng.sign_bits >> j) & 1 else 1 for j in range(32)])
    ref2 = oracle.quantize(to_oracle(x), 32, signs=signs, mode=oracle.ABSMAX_RTN, want_mask=True, want_dequant=True)
    assert np.array_equal(to_oracle(deq), ref2["dequant"])
    assert np.array_equal(clip.cpu().numpy(), oracle.unpack_mask(ref2["mask"]))
    assert np.array_equal(to_oracle(tseng(x.to(dev))), ref2["dequant"])
    aligned = q.AlignedAlbertTsengQuantizer()
    got = aligned(x.to(dev)).float().cpu().numpy()
    base = oracle.bf16_bits_to_f32(oracle.quantize(to_oracle(x), 32, mode=oracle.ABSMAX_RTN, want_dequant=True)["dequant"])
    np.testing.assert_allclose(got, base * 1.009276, rtol=2 ** -7)


def test_notebook_error_bands_on_gpu(q):
    # notebooks/benchmark_mxfp4.ipynb: x = randn(1,128,4096), w = randn(128,4096) bf16, deterministic
    # backward: 2e-2 < fwd rel^2 err < 6e-2 and 6e-2 < wgrad rel^2 err < 15e-2 against plain bf16 linear
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, 128, 4096, generator=g).to(torch.bfloat16).to("cuda:0").requires_grad_(True)
    w = torch.randn(128, 4096, generator=g).to(torch.bfloat16).to("cuda:0")
    dy = torch.randn(1, 128, 128, generator=g).to(torch.bfloat16).to("cuda:0")
    layer = production_layer(q, 4096, 128, False, None, torch.bfloat16)
    with torch.no_grad():
        layer.weight.copy_(w)
    y = layer(x)
    y.backward(dy)
    wref = w.clone().float().requires_grad_(True)
    yref = torch.nn.functional.linear(x.detach().float(), wref)
    yref.backward(dy.float())
    err = lambda a, b: float(((a.detach().float() - b.detach().float()) ** 2).sum() / (b.detach().float() ** 2).sum())
    assert 2e-2 < err(y, yref) < 6e-2
    assert 6e-2 < err(layer.weight.grad, wref.grad) < 15e-2


@pytest.mark.parametrize("cls_name,mode_name,post", [("QuestMXFP4Quantizer", "QUEST_RTN", 1.0),
                                                     ("AlbertTsengQuantizer", "ABSMAX_SR", 1.0),
                                                     ("AlignedAlbertTsengQuantizer", "ABSMAX_RTN", 1.009276)])
def test_dense_rotation_quantizers_against_oracle(oracle, q, cls_name, mode_name, post):
    """rerotate="O32": the kernel rotates every group of 32 by the module's dense matrix and quantizes it; the oracle
    with the same matrix must give the same pseudo-quantized values bit for bit, and the backward pass is the (masked)
    product with the transposed matrix."""
    print(f"case dense rotation {cls_name}", flush=True)
    import random
    dev = "cuda:0"
    torch.manual_seed(11)
    quant = getattr(q, cls_name)(hadamard_dim=32, rerotate="O32")
    quant.re_randomize()
    x = make_input(48, 256, torch.bfloat16, seed=12).to(dev).requires_grad_(True)
    random.seed(4)
    y = quant(x)
    R = quant.hadamard_matrix
    assert R.dtype == torch.bfloat16 and R.device.type == "cuda"
    random.seed(4)
    seed = random.getrandbits(63) if "SR" in mode_name else 0
    want = oracle.quantize(to_oracle(x.detach()), mode=getattr(oracle, mode_name), seed=seed, want_mask=True, want_dequant=True,
                           matrix=quant._dense.numpy())
    from tests.util import from_oracle_bf16
    ref = from_oracle_bf16(want["dequant"])
    if post != 1.0:
        ref = ref * post   # the module scales the kernel's bf16 result in place
    assert torch.equal(y.detach().cpu(), ref)
    g = make_input(48, 256, torch.bfloat16, seed=13).to(dev)
    y.backward(g)
    gm = g.float()
    if cls_name == "QuestMXFP4Quantizer":
        bits = torch.from_numpy(np.unpackbits(want["mask"], axis=1, bitorder="little")).to(dev).float()
        gm = gm * bits
    gref = (gm.reshape(-1, 32) @ R.float().T).view(48, 256)
    assert float((x.grad.float() - gref).norm() / gref.norm()) < 1e-2   # the module's product runs in bf16


@pytest.mark.parametrize("hd", [64, 128])
@pytest.mark.parametrize("cls_name,mode_name", [("QuestMXFP4Quantizer", "QUEST_RTN"), ("AlbertTsengQuantizer", "ABSMAX_SR")])
def test_dense_rotation_over_wider_blocks(oracle, q, hd, cls_name, mode_name):
    """rerotate="O32" with hadamard_dim 64 / 128: the module holds an [hd, hd] orthogonal matrix (mxfp4.py:61-64), applies
    it as an fp32 product and hands the rotated rows to the kernel as they are.  Forward equals the oracle's quantizer on
    the same rotated tensor bit for bit; backward is the (masked) product with the transposed matrix."""
    print(f"case dense rotation hd={hd} {cls_name}", flush=True)
    import random
    from tests.util import from_oracle_bf16
    dev = "cuda:0"
    torch.manual_seed(21)
    quant = getattr(q, cls_name)(hadamard_dim=hd, rerotate="O32")
    quant.re_randomize()
    assert quant.is_dense and quant._dense.shape == (hd, hd)
    x = make_input(40, 256, torch.bfloat16, seed=22).to(dev).requires_grad_(True)
    random.seed(9)
    y = quant(x)
    R = quant.hadamard_matrix
    assert R.shape == (hd, hd) and R.dtype == torch.bfloat16
    rotated = (x.detach().reshape(-1, hd).float() @ R.float()).view(40, 256)
    random.seed(9)
    seed = random.getrandbits(63) if "SR" in mode_name else 0
    want = oracle.quantize(to_oracle(rotated), hd=1, mode=getattr(oracle, mode_name), seed=seed, want_mask=True, want_dequant=True)
    ref = torch.from_numpy(want["dequant"]).to(torch.bfloat16)      # de-quantized values are exact in bf16
    assert y.dtype == torch.bfloat16 and torch.equal(y.detach().cpu(), ref)
    g = make_input(40, 256, torch.bfloat16, seed=23).to(dev)
    y.backward(g)
    gm = g.float()
    if cls_name == "QuestMXFP4Quantizer":
        gm = gm * torch.from_numpy(np.unpackbits(want["mask"], axis=1, bitorder="little")).to(dev).float()
    gref = (gm.reshape(-1, hd) @ R.float().T).view(40, 256)
    assert float((x.grad.float() - gref).norm() / gref.norm()) < 1e-2   # the module's product runs in bf16


def test_layer_with_dense_gradient_rotation(oracle, q):
    """The production configuration with rerotate="O32" on the gradient quantizer stays on the packed FP4 path (the
    four gradient quantizations rotate by the dense matrix on the matrix pipe): the step must equal the oracle pipeline
    with the same matrix and seeds, and gradients stay as close to the unquantized ones as with sign flips."""
    print("case layer with O32 gradient rotation", flush=True)
    T, I, O = 256, 512, 128
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, I, generator=g).to(torch.bfloat16)
    w = torch.randn(O, I, generator=g).to(torch.bfloat16)
    dy = torch.randn(T, O, generator=g).to(torch.bfloat16)
    wref = w.clone().float().requires_grad_(True)
    xref = x.clone().float().requires_grad_(True)
    torch.nn.functional.linear(xref, wref).backward(dy.float())
    err = lambda a, b: float(((a.detach().float().cpu() - b.detach().float()) ** 2).sum() / (b.detach().float() ** 2).sum())
    errs = {}
    for rr in ("signs", "O32"):
        torch.manual_seed(1)
        random.seed(9)
        layer = production_layer(q, I, O, True, rr, torch.bfloat16)
        assert layer._is_production_config(T)
        with torch.no_grad():
            layer.weight.copy_(w)
        xin = x.clone().to("cuda:0").requires_grad_(True)
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            y = layer(xin)
        y.backward(dy.to("cuda:0"))
        g_q = layer.backward_scheme.g_quantizer
        assert g_q.is_dense == (rr == "O32")
        errs[rr] = (err(xin.grad, xref.grad), err(layer.weight.grad, wref.grad))
        if rr == "O32":
            # the oracle pipeline with the matrix the layer drew and the seeds it used
            random.seed(9)
            seeds = [random.getrandbits(63) for _ in range(4)]
            H = g_q._dense.numpy()
            d = float(oracle.FOUR_THIRDS)
            qx = oracle.quantize(to_oracle(x), 32, mode=oracle.QUEST_RTN, want_mask=True)
            qw = oracle.quantize(to_oracle(w), 32, mode=oracle.QUEST_RTN, want_mask=True)
            qe = oracle.quantize(to_oracle(dy), mode=oracle.ABSMAX_SR, seed=seeds[0], matrix=H)
            qwt = oracle.requantize_transposed(qw["codes"], qw["scales"], val_dtype=oracle.BF16, mode=oracle.ABSMAX_SR, seed=seeds[1], matrix=H)
            gxq = oracle.gemm_tn(qe["codes"], qe["scales"], qwt["codes"], qwt["scales"], a_post=d, b_post=d)
            qet = oracle.quantize(to_oracle(dy), mode=oracle.ABSMAX_SR, transposed_in=True, seed=seeds[2], matrix=H)
            qxt = oracle.requantize_transposed(qx["codes"], qx["scales"], val_dtype=oracle.BF16, mode=oracle.ABSMAX_SR, seed=seeds[3], matrix=H)
            gwq = oracle.gemm_tn(qet["codes"], qet["scales"], qxt["codes"], qxt["scales"], a_post=d, b_post=d)
            from tests.util import from_oracle_bf16
            gx_ref = from_oracle_bf16(oracle.masked_hadamard_bwd(to_oracle(torch.from_numpy(gxq).to(torch.bfloat16)), 32, oracle.BF16, None, qx["mask"]))
            gw_ref = from_oracle_bf16(oracle.masked_hadamard_bwd(to_oracle(torch.from_numpy(gwq).to(torch.bfloat16)), 32, oracle.BF16, None, qw["mask"]))
            assert rel(xin.grad.float().cpu(), gx_ref.float()) < 1e-2
            assert rel(layer.weight.grad.float().cpu(), gw_ref.float()) < 1e-2
    print(f"relative squared gradient errors {errs}", flush=True)
    for k in (0, 1):
        assert 0.03 < errs["O32"][k] < 0.3 and abs(errs["O32"][k] - errs["signs"][k]) < 0.5 * errs["signs"][k]


@pytest.mark.parametrize("dense", ["x", "w", "xw"])
@pytest.mark.parametrize("dtype,shape", [(torch.float32, (384, 256, 160)), (torch.bfloat16, (384, 256, 160)),
                                         (torch.bfloat16, (256, 512, 256))])
def test_layer_with_dense_forward_rotation(oracle, q, dense, dtype, shape):
    """A forward quantizer that holds the dense matrix of rerotate="O32" (mxfp4.py:61-64) keeps the layer on the packed
    FP4 path: the dense quantizer kernel fills the packed operand, the gradient products run as ever, and the
    straight-through backward is (g * clip mask) @ matrix^T (mxfp4.py:143-146).  Checked against the oracle pipeline
    with the matrices the quantizers drew, on the row-major and the tiled operand layout, and against the module path."""
    print(f"case layer with dense forward rotation of {dense} dtype={dtype} shape={shape}", flush=True)
    T, I, O = shape
    x = make_input(T, I, dtype, seed=1, outlier_frac=0.01)
    w = make_input(O, I, dtype, seed=2, outlier_frac=0, scale=0.02)
    dy = make_input(T, O, dtype, seed=3, outlier_frac=0, scale=1e-3)
    layer = production_layer(q, I, O, True, None, dtype)
    torch.manual_seed(11)
    mats = {}
    for name, quantizer in (("x", layer.activation_quantizer), ("w", layer.weight_quantizer)):
        if name in dense:
            quantizer.rerotate = "O32"
            quantizer.re_randomize()
            assert quantizer.is_dense
            mats[name] = quantizer._dense.to(dtype).double().numpy()   # the modules cast the matrix to the tensor's dtype
    assert layer._is_production_config(T)
    with torch.no_grad():
        layer.weight.copy_(w.to("cuda:0"))

    def step(packed):
        layer.use_packed_path = packed
        layer.weight.grad = None
        xd = x.to("cuda:0").requires_grad_(True)
        random.seed(5)
        y = layer(xd)
        y.backward(dy.to("cuda:0"))
        torch.cuda.synchronize()
        return y.detach().float().cpu().numpy(), xd.grad.float().cpu().numpy(), layer.weight.grad.float().cpu().numpy(), xd.grad.dtype

    y, gx, gw, gdt = step(True)
    assert gdt == dtype
    random.seed(5)
    seeds = [random.getrandbits(63) for _ in range(4)]
    vd = oracle.BF16 if dtype == torch.bfloat16 else oracle.F32
    d = float(oracle.FOUR_THIRDS)
    fwd = lambda t, name: (oracle.quantize(to_oracle(t), mode=oracle.QUEST_RTN, want_mask=True, matrix=mats[name].astype(np.float32))
                           if name in dense else oracle.quantize(to_oracle(t), 32, mode=oracle.QUEST_RTN, want_mask=True))
    qx, qw = fwd(x, "x"), fwd(w, "w")
    y_ref = oracle.gemm_tn(qx["codes"], qx["scales"], qw["codes"], qw["scales"])
    qe = oracle.quantize(to_oracle(dy), 32, mode=oracle.ABSMAX_SR, seed=seeds[0])
    qwt = oracle.requantize_transposed(qw["codes"], qw["scales"], val_dtype=vd, hd=32, mode=oracle.ABSMAX_SR, seed=seeds[1])
    gxq = oracle.gemm_tn(qe["codes"], qe["scales"], qwt["codes"], qwt["scales"], a_post=d, b_post=d)
    qet = oracle.quantize(to_oracle(dy), 32, mode=oracle.ABSMAX_SR, transposed_in=True, seed=seeds[2])
    qxt = oracle.requantize_transposed(qx["codes"], qx["scales"], val_dtype=vd, hd=32, mode=oracle.ABSMAX_SR, seed=seeds[3])
    gwq = oracle.gemm_tn(qet["codes"], qet["scales"], qxt["codes"], qxt["scales"], a_post=d, b_post=d)

    def ste(gq, packed, name):
        if name not in dense:
            return oracle.masked_hadamard_bwd(gq.astype(np.float32), 32, vd, None, packed["mask"], out_dtype=oracle.F32)
        keep = np.unpackbits(packed["mask"], axis=1, bitorder="little").astype(np.float64)
        return ((gq * keep).reshape(-1, 32) @ mats[name].T).reshape(gq.shape)

    tol_y, tol_g = (1e-5, 1e-5) if dtype == torch.float32 else (3e-3, 6e-3)
    assert rel(y, y_ref) <= tol_y
    assert rel(gx, ste(gxq, qx, "x")) <= tol_g
    assert rel(gw, ste(gwq, qw, "w")) <= tol_g
    # the module path (quantizer modules, de-quantized tensors, library products) computes the same forward pass; its
    # backward draws its seeds in another order, so only the size of the difference is checked there
    y_mod, gx_mod, gw_mod, _ = step(False)
    assert rel(y_mod, y) <= (1e-5 if dtype == torch.float32 else 6e-3)
    assert rel(gx_mod, gx) < 1.0 and rel(gw_mod, gw) < 1.0


@pytest.mark.parametrize("dense", ["x", "w", "xw"])
def test_dense_forward_rotation_under_autocast(q, dense):
    """fp32 master weights under bf16 autocast (the Llama configurations) with dense forward rotations and a deterministic
    backward: the packed path and the module path (quantizer modules, de-quantized tensors, library products) agree on
    the output and on both gradients to the bf16 roundings they place differently; gradients keep the parameters' dtypes."""
    print(f"case dense forward rotation under autocast, dense={dense}", flush=True)
    T, I, O = 256, 384, 256
    x = make_input(T, I, torch.float32, seed=1, outlier_frac=0.01)
    w = make_input(O, I, torch.float32, seed=2, outlier_frac=0, scale=0.02)
    dy = make_input(T, O, torch.bfloat16, seed=3, outlier_frac=0, scale=1e-3)
    layer = production_layer(q, I, O, False, None, torch.float32)
    torch.manual_seed(7)
    for name, quantizer in (("x", layer.activation_quantizer), ("w", layer.weight_quantizer)):
        if name in dense:
            quantizer.rerotate = "O32"
            quantizer.re_randomize()
    with torch.no_grad():
        layer.weight.copy_(w.to("cuda:0"))
    outs = []
    for packed in (True, False):
        layer.use_packed_path = packed
        layer.weight.grad = None
        xd = x.to("cuda:0").requires_grad_(True)
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):   # around forward and backward, as the training loop has it
            y = layer(xd)
            y.backward(dy.to("cuda:0"))
        assert y.dtype == torch.bfloat16 and xd.grad.dtype == torch.float32 and layer.weight.grad.dtype == torch.float32
        outs.append((y.detach().float().cpu().numpy(), xd.grad.cpu().numpy(), layer.weight.grad.cpu().numpy()))
    layer.use_packed_path = True
    assert layer._is_production_config(T)
    for got, want, tol in zip(outs[0], outs[1], (6e-3, 2e-2, 2e-2)):
        assert rel(got, want) <= tol


def test_packed_weight_cache_across_micro_steps(q):
    """With the cache on, the second micro-step reuses the packed Q(W) of the first: outputs and gradients are
    bit-identical to a layer that quantizes every time, the buffer saved by an earlier graph survives a weight
    update, and an update (seen through the version counter, or announced by invalidate) re-quantizes."""
    torch.manual_seed(5)
    T, I, O = 256, 256, 384
    cached = production_layer(q, I, O, False, None, torch.bfloat16)
    plain = production_layer(q, I, O, False, None, torch.bfloat16)
    with torch.no_grad():
        plain.weight.copy_(cached.weight)
    q.enable_packed_weight_cache(cached)
    cache = cached.packed_weight_cache
    assert plain.packed_weight_cache is None and cache.hits == 0

    def step(layer, x, dy):
        x = x.clone().requires_grad_(True)
        layer.weight.grad = None
        y = layer(x)
        y.backward(dy)
        return y.detach(), x.grad, layer.weight.grad

    xs = [make_input(T, I, torch.bfloat16, seed=s).to("cuda:0") for s in (1, 2, 3)]
    dys = [make_input(T, O, torch.bfloat16, seed=10 + s).to("cuda:0") for s in (1, 2, 3)]
    for k in (0, 1):
        for got, want in zip(step(cached, xs[k], dys[k]), step(plain, xs[k], dys[k])):
            assert torch.equal(got, want)
    assert (cache.misses, cache.hits) == (1, 1)
    first_buffer = cache.buffer

    # a graph built before the update still owns the old Q(W) when its backward runs after the update
    x_old = xs[0].clone().requires_grad_(True)
    y_old = cached(x_old)
    assert cache.hits == 2
    with torch.no_grad():
        cached.weight.mul_(0.5)
        plain.weight.mul_(0.5)
    for got, want in zip(step(cached, xs[2], dys[2]), step(plain, xs[2], dys[2])):
        assert torch.equal(got, want)
    assert cache.misses == 2 and cache.buffer is not first_buffer
    y_old.backward(dys[0])
    with torch.no_grad():
        plain.weight.mul_(2.0)      # powers of two: exactly the old weight again
    _, gx_want, _ = step(plain, xs[0], dys[0])
    assert torch.equal(x_old.grad, gx_want)

    # an update that the version counter does not see has to be announced
    with torch.no_grad():
        plain.weight.copy_(cached.weight)
    cached.weight.data.mul_(2.0)
    plain.weight.data.mul_(2.0)
    q.invalidate_packed_weights(cached)
    for got, want in zip(step(cached, xs[1], dys[1]), step(plain, xs[1], dys[1])):
        assert torch.equal(got, want)
    assert cache.misses == 3


@pytest.mark.parametrize("T,I,O", [(256, 256, 384), (64, 96, 160)])
def test_weight_gradient_widened_in_the_kernel(q, T, I, O):
    """gw_dtype = float32 with bf16 intermediates: the last kernel of the backward pass writes the bf16-rounded weight
    gradient as fp32 -- the bits a separate bf16 -> fp32 conversion of the bf16 result holds."""
    from quartet_amd import kernels as K
    x = make_input(T, I, torch.bfloat16, seed=1).to("cuda:0")
    w = make_input(O, I, torch.float32, seed=2, scale=0.02).to("cuda:0")
    e = make_input(T, O, torch.bfloat16, seed=3, scale=1e-2, outlier_frac=0).to("cuda:0")
    tiled = all(d % 128 == 0 and d >= 256 for d in (T, I, O))
    _, px, pw = K.linear_forward(x, w, 32, 0x5A5A5A5A, 32, 0x0F0F1234, torch.bfloat16, tiled)
    args = (e, px, pw, T, I, O, 32, 0x5A5A5A5A, 32, 0x0F0F1234, 32, 0x13572468, K.QM_ABSMAX_SR, [11, 12, 13, 14],
            torch.bfloat16, torch.float32, torch.bfloat16, torch.bfloat16, torch.bfloat16, tiled)
    gx0, gw0 = K.linear_backward(*args)
    gx1, gw1 = K.linear_backward(*args, gw_dtype=torch.float32)
    assert gw0.dtype == torch.bfloat16 and gw1.dtype == torch.float32
    assert torch.equal(gx0, gx1) and torch.equal(gw0.float(), gw1)
    gx2, gw2 = K.linear_backward(*args, gx_rotated=True, gw_dtype=torch.float32)
    assert torch.equal(gw2, gw1)
    mask = K.packed_mask_bits(px, T, I)
    assert torch.equal(K.masked_hadamard_bwd(gx2, 32, torch.bfloat16, 0x5A5A5A5A, mask), gx0)


@pytest.mark.parametrize("mid_dtype,gw_dtype", [(torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32),
                                                (torch.float32, torch.float32)])
def test_backward_with_products_cut_into_k_ranges(q, mid_dtype, gw_dtype):
    """Few output tiles and a long contraction: both gradient products are cut into K ranges, and the ordered reduction of
    the ranges applies the masked inverse rotation in the same pass.  Bit for bit what the kernels give one by one
    (quantizers, re-quantizers, the products with their plain reduction, the inverse rotation as a kernel of its own)."""
    print(f"case backward with split products mid={mid_dtype} gw={gw_dtype}", flush=True)
    from quartet_amd import kernels as K
    from quartet_amd import _lib
    T, I, O = 4096, 512, 2048
    assert _lib.lib().qm_gemm_workspace_bytes(T, I, O) > 0 and _lib.lib().qm_gemm_workspace_bytes(O, I, T) > 0
    dev = "cuda:0"
    x = make_input(T, I, mid_dtype, seed=21).to(dev)
    w = make_input(O, I, mid_dtype, seed=22, scale=0.02).to(dev)
    e = make_input(T, O, mid_dtype, seed=23, scale=1e-2, outlier_frac=0).to(dev)
    sx, sw, sg, seeds, tl = 0x5A5A5A5A, 0x0F0F1234, 0x13572468, [11, 12, 13, 14], True
    _, px, pw = K.linear_forward(x, w, 32, sx, 32, sw, mid_dtype, tl)
    gx, gw = K.linear_backward(e, px, pw, T, I, O, 32, sx, 32, sw, 32, sg, K.QM_ABSMAX_SR, seeds, mid_dtype, mid_dtype, mid_dtype,
                               mid_dtype, mid_dtype, tl, gw_dtype=gw_dtype)
    assert gx.dtype == mid_dtype and gw.dtype == gw_dtype
    alpha = float(torch.tensor(K.FOUR_THIRDS, dtype=torch.float32) * torch.tensor(K.FOUR_THIRDS, dtype=torch.float32))
    xc, xs, xm, _ = K.quantize_mxfp4(x, 32, sx, K.QM_QUEST_RTN, want_mask=True, tiled=tl)
    wc, ws, wm, _ = K.quantize_mxfp4(w, 32, sw, K.QM_QUEST_RTN, want_mask=True, tiled=tl)
    ec, es, _, _ = K.quantize_mxfp4(e, 32, sg, K.QM_ABSMAX_SR, seed=seeds[0], tiled=tl)
    wtc, wts, _ = K.requantize_transposed_mxfp4(wc, ws, 1.0, mid_dtype, 32, sg, K.QM_ABSMAX_SR, seed=seeds[1], tiled_in=tl, tiled_out=tl)
    etc, ets, _, _ = K.quantize_mxfp4(e, 32, sg, K.QM_ABSMAX_SR, transposed_in=True, seed=seeds[2], tiled=tl)
    xtc, xts, _ = K.requantize_transposed_mxfp4(xc, xs, 1.0, mid_dtype, 32, sg, K.QM_ABSMAX_SR, seed=seeds[3], tiled_in=tl, tiled_out=tl)
    gxq = K.gemm_mxfp4_tn(ec, es, wtc, wts, alpha, mid_dtype, a_tiled=tl, b_tiled=tl, split_k=True)
    gwq = K.gemm_mxfp4_tn(etc, ets, xtc, xts, alpha, mid_dtype, a_tiled=tl, b_tiled=tl, split_k=True)
    assert torch.equal(gx, K.masked_hadamard_bwd(gxq, 32, mid_dtype, sx, xm))
    want_gw = K.masked_hadamard_bwd(gwq, 32, mid_dtype, sw, wm)
    assert torch.equal(gw, want_gw.to(gw_dtype))
    assert gw.abs().max() > 0 and gx.abs().max() > 0


@pytest.mark.parametrize("three_d", [False, True])
@pytest.mark.parametrize("stochastic", [False, True])
def test_error_only_scheme_against_oracle(oracle, q, three_d, stochastic):
    """Scheme "Q(E)W_Q(Et)X" (src/models/quantization/backward.py:21-45 of the reference): only the error signal is
    quantized; grad_x = Q(e) W and grad_W = Q(e^T) x with the saved operands as they are.  Checked against the oracle's
    de-quantized Q(e), Q(e^T) (same seeds, same accumulated sign flips) multiplied in float64, for a 2-D and a 3-D
    input."""
    print(f"case scheme Q(E)W_Q(Et)X three_d={three_d} stochastic={stochastic}", flush=True)
    dev = "cuda:0"
    B, S, I, O = 4, 96, 256, 160
    g_q = q.AlbertTsengQuantizer(stochastic=stochastic, rerotate="signs")
    torch.manual_seed(5)
    g_q.re_randomize()   # the scheme itself never re-randomises (the reference's does not either)
    signs = np.array([-1 if (g_q.sign_bits >> j) & 1 else 1 for j in range(32)])
    layer = q.QuantizedLinear(I, O, bias=False, gradient_quantizer=g_q,
                              backward_scheme=q.BACKWARD_SCHEMES["Q(E)W_Q(Et)X"]()).to(dev)
    assert type(layer.backward_scheme).__name__ == "QEW_QEtX_Scheme" and layer.backward_scheme.g_quantizer is g_q
    x = make_input(B * S, I, torch.float32, 31, outlier_frac=0.0)
    dy = make_input(B * S, O, torch.float32, 32, outlier_frac=0.0, scale=1e-3)
    w = layer.weight.detach().cpu()
    shape = (B, S) if three_d else (B * S,)
    xd = x.view(*shape, I).to(dev).requires_grad_(True)
    y = layer(xd)
    assert y.shape == (*shape, O)
    assert rel(y.detach().cpu().view(-1, O), x.double() @ w.double().T) < 1e-5   # identity quantizers in the forward pass
    random.seed(77)
    y.backward(dy.view(*shape, O).to(dev))
    torch.cuda.synchronize()
    random.seed(77)
    seeds = [random.getrandbits(63) for _ in range(2)] if stochastic else [0, 0]
    mode = oracle.ABSMAX_SR if stochastic else oracle.ABSMAX_RTN
    qe = oracle.quantize(to_oracle(dy), 32, signs=signs, mode=mode, seed=seeds[0], want_dequant=True)
    qet = oracle.quantize(to_oracle(dy), 32, signs=signs, mode=mode, transposed_in=True, seed=seeds[1], want_dequant=True)
    gx_ref = qe["dequant"].astype(np.float64) @ w.double().numpy()
    gw_ref = qet["dequant"].astype(np.float64) @ x.double().numpy()
    assert xd.grad.shape == xd.shape and layer.weight.grad.shape == (O, I)
    assert rel(xd.grad.cpu().view(-1, I), gx_ref) < 1e-5
    assert rel(layer.weight.grad.cpu(), gw_ref) < 1e-5
    # The MXFP4 quantizers return the tensor in the rotated basis (the reference's kernel never rotates back), so this
    # scheme multiplies the rotated Q(e) with the unrotated W exactly as the reference does: the product is close to
    # (e H) W, FP4 noise apart, not to e W.
    rot = oracle.quantize(to_oracle(dy), 32, signs=signs, mode=oracle.ABSMAX_RTN, want_rotated=True)["rotated"]
    assert 0.02 < rel(gx_ref, rot.astype(np.float64) @ w.double().numpy()) < 0.3


def test_error_only_scheme_under_autocast(oracle, q):
    """The same scheme the way the training loop runs it: bf16 autocast around forward and backward, so the products are
    bf16 library GEMMs on the de-quantized bf16 Q(e)."""
    print("case scheme Q(E)W_Q(Et)X under bf16 autocast", flush=True)
    dev = "cuda:0"
    T, I, O = 512, 384, 256
    layer = q.QuantizedLinear(I, O, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
                              activation_quantizer=q.QuestMXFP4Quantizer(),
                              gradient_quantizer=q.AlbertTsengQuantizer(stochastic=False),
                              backward_scheme=q.BACKWARD_SCHEMES["Q(E)W_Q(Et)X"]()).to(dev)
    x = make_input(T, I, torch.bfloat16, 41, outlier_frac=0.0)
    dy = make_input(T, O, torch.bfloat16, 42, outlier_frac=0.0, scale=1e-3)
    xd = x.to(dev).requires_grad_(True)
    with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
        y = layer(xd)
        y.backward(dy.to(dev))
    torch.cuda.synchronize()
    qx = oracle.quantize(to_oracle(x), 32, mode=oracle.QUEST_RTN, want_mask=True, want_dequant=True)
    qw = oracle.quantize(to_oracle(layer.weight.detach().cpu()), 32, mode=oracle.QUEST_RTN, want_mask=True, want_dequant=True)
    qe = oracle.quantize(to_oracle(dy), 32, mode=oracle.ABSMAX_RTN, want_dequant=True)
    qet = oracle.quantize(to_oracle(dy), 32, mode=oracle.ABSMAX_RTN, transposed_in=True, want_dequant=True)
    from tests.util import from_oracle_bf16
    # the scheme multiplies Q(e) with the saved pseudo-quantized operands (bf16 under autocast), then the forward
    # quantizers' straight-through backward (clip mask + inverse rotation) maps the results to x and W
    wq = qw["dequant"].astype(np.float64)
    xq = from_oracle_bf16(qx["dequant"]).double().numpy()
    eq, etq = from_oracle_bf16(qe["dequant"]).double().numpy(), from_oracle_bf16(qet["dequant"]).double().numpy()
    gxq = torch.from_numpy(eq @ torch.from_numpy(wq).to(torch.bfloat16).double().numpy()).to(torch.bfloat16)
    gwq = torch.from_numpy(etq @ xq).to(torch.bfloat16)
    gx_ref = from_oracle_bf16(oracle.masked_hadamard_bwd(to_oracle(gxq), 32, oracle.BF16, None, qx["mask"])).double().numpy()
    gw_ref = from_oracle_bf16(oracle.masked_hadamard_bwd(to_oracle(gwq), 32, oracle.BF16, None, qw["mask"])).double().numpy()
    assert rel(xd.grad.float().cpu(), gx_ref) < 1e-2
    assert rel(layer.weight.grad.float().cpu(), gw_ref) < 1e-2


@pytest.mark.parametrize("cls_name,stochastic", [("AlbertTsengQuantizer", True), ("AlbertTsengQuantizer", False),
                                                 ("AlignedAlbertTsengQuantizer", False), ("QuestMXFP4Quantizer", False)])
def test_error_only_scheme_on_packed_codes(oracle, q, cls_name, stochastic, monkeypatch):
    """Scheme "Q(E)W_Q(Et)X" with bf16 products (autocast): grad_x = Q(e) w and grad_w = Q(e^T) x run on the packed codes
    of Q(e) in the FP4 x bf16 kernel (both products, counted), with the saved operands as they lie in memory.  Checked
    against the oracle's de-quantized Q(e), Q(e^T) (same seeds) times the bf16 operands in float64; the only rounding
    beyond fp32 accumulation is the bf16 output (2^-9 per element)."""
    print(f"case packed error-only scheme {cls_name} stochastic={stochastic}", flush=True)
    from quartet_amd import kernels as K
    dev = "cuda:0"
    T, I, O = 384, 200, 192
    kw = {"stochastic": stochastic} if cls_name == "AlbertTsengQuantizer" else {}
    g_q = getattr(q, cls_name)(**kw)
    layer = q.QuantizedLinear(I, O, bias=False, gradient_quantizer=g_q, backward_scheme=q.BACKWARD_SCHEMES["Q(E)W_Q(Et)X"]()).to(dev)
    calls = []
    real = K.gemm_mxfp4_bf16_nn
    monkeypatch.setattr(K, "gemm_mxfp4_bf16_nn", lambda *a, **k: (calls.append(a[2].shape), real(*a, **k))[1])
    x = make_input(T, I, torch.bfloat16, 51, outlier_frac=0.0)
    dy = make_input(T, O, torch.bfloat16, 52, outlier_frac=0.0, scale=1e-3)
    xd = x.to(dev).requires_grad_(True)
    random.seed(91)
    with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
        y = layer(xd)
        y.backward(dy.to(dev))
    torch.cuda.synchronize()
    assert calls == [(O, I), (T, I)]
    random.seed(91)
    seeds = [random.getrandbits(63) for _ in range(2)] if stochastic else [0, 0]
    mode = {"QuestMXFP4Quantizer": oracle.QUEST_RTN}.get(cls_name, oracle.ABSMAX_SR if stochastic else oracle.ABSMAX_RTN)
    post = 1.009276 if cls_name == "AlignedAlbertTsengQuantizer" else 1.0
    qe = oracle.quantize(to_oracle(dy), 32, mode=mode, seed=seeds[0])
    qet = oracle.quantize(to_oracle(dy), 32, mode=mode, transposed_in=True, seed=seeds[1])
    d = 1.0 if mode == oracle.QUEST_RTN else float(oracle.FOUR_THIRDS)
    w16 = layer.weight.detach().to(torch.bfloat16).double().cpu().numpy()
    gx_ref = post * oracle.dequantize(qe["codes"], qe["scales"], d).astype(np.float64) @ w16
    gw_ref = post * oracle.dequantize(qet["codes"], qet["scales"], d).astype(np.float64) @ x.double().numpy()
    assert xd.grad.shape == (T, I) and layer.weight.grad.shape == (O, I)
    assert rel(xd.grad.float().cpu(), gx_ref) < 3e-3
    assert rel(layer.weight.grad.float().cpu(), gw_ref) < 3e-3


def test_error_only_scheme_keeps_the_library_path_for_fp32_products(q, monkeypatch):
    """Without autocast on fp32 tensors the reference's products are fp32 library GEMMs: the packed kernel (bf16 operand)
    must not be used."""
    from quartet_amd import kernels as K
    monkeypatch.setattr(K, "gemm_mxfp4_bf16_nn", lambda *a, **k: pytest.fail("packed product used for fp32 operands"))
    dev = "cuda:0"
    layer = q.QuantizedLinear(128, 64, bias=False, gradient_quantizer=q.AlbertTsengQuantizer(stochastic=False),
                              backward_scheme=q.BACKWARD_SCHEMES["Q(E)W_Q(Et)X"]()).to(dev)
    x = torch.randn(64, 128, device=dev, requires_grad=True)
    layer(x).sum().backward()
    assert torch.isfinite(x.grad).all() and torch.isfinite(layer.weight.grad).all()
