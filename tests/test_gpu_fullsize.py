"""Parity at the benchmark's full sizes (tokens 8192, features 4096; the quantizer also at 65536 x 4096), where the
CPU oracle cannot process whole tensors in test time.  Each check is a size-independent property that reduces
to an oracle comparison on a slice:

* row-major quantization is row-local, so any subset of rows of the big result must equal the oracle's result on
  those rows (round-to-nearest modes), and the leading rows also with the in-kernel random stream, whose
  counters are flat element offsets and therefore identical for a prefix;
* the transposed and re-quantizing kernels are local to a column of their input, so a 32-column slice of the
  input gives 32 complete output rows;
* every output row of a GEMM depends on one row of A only: rows of the full product equal the product of those
  rows alone, and a sample is checked against the float64 product of the de-quantized operands;
* tiled and row-major code bytes are permutations of each other."""
import numpy as np
import pytest
import torch

from tests.util import to_oracle

pytestmark = pytest.mark.gpu

T, I, O = 8192, 4096, 4096


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from quartet_amd import kernels
    return kernels


@pytest.fixture(scope="module")
def data():
    g = torch.Generator().manual_seed(123)
    x = torch.randn(T, I, generator=g)
    heavy = torch.rand(T, I, generator=g) < 0.01
    x = torch.where(heavy, 30.0 * torch.randn(T, I, generator=g), x).to(torch.bfloat16)
    dy = (1e-3 * torch.randn(T, O, generator=g)).to(torch.bfloat16)
    return x, dy


def _rows(t, idx):
    return to_oracle(t[idx])


@pytest.mark.parametrize("rows", [T, 65536])
@pytest.mark.parametrize("mode,want_mask", [(0, True), (1, False)])
def test_rowmajor_sampled_rows_match_oracle(oracle, K, rows, mode, want_mask):
    print(f"case fullsize rowmajor rows={rows} mode={mode}", flush=True)
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(rows + mode)
    gd = torch.Generator(device=dev).manual_seed(rows + mode)
    xd = torch.randn(rows, I, generator=gd, device=dev)
    xd[torch.rand(rows, I, generator=gd, device=dev) < 1e-3] = 1e3
    xd = xd.to(torch.bfloat16)
    signs = 0x9D2C5681
    codes, scales, mask, _ = K.quantize_mxfp4(xd, 32, signs, mode, want_mask=want_mask)
    tcodes, tscales, tmask, _ = K.quantize_mxfp4(xd, 32, signs, mode, want_mask=want_mask, tiled=True)
    torch.cuda.synchronize()
    assert torch.equal(K.untile_codes(tcodes), codes) and torch.equal(tscales, scales)
    if want_mask:
        assert torch.equal(tmask, mask)
    idx = torch.cat([torch.arange(0, 32), torch.randint(0, rows, (96,), generator=g), torch.arange(rows - 16, rows)])
    sv = np.array([-1 if (signs >> j) & 1 else 1 for j in range(32)])
    ref = oracle.quantize(to_oracle(xd[idx.to(dev)]), 32, signs=sv, mode=mode, want_mask=want_mask)
    assert np.array_equal(_rows(codes, idx.to(dev)), ref["codes"])
    assert np.array_equal(_rows(scales, idx.to(dev)), ref["scales"])
    if want_mask:
        assert np.array_equal(_rows(mask, idx.to(dev)), ref["mask"])
    # row locality: permuting rows permutes the result
    perm = torch.randperm(rows, generator=g)[:4096].to(dev)
    pc, ps, _, _ = K.quantize_mxfp4(xd[perm].contiguous(), 32, signs, mode)
    assert torch.equal(pc, codes[perm]) and torch.equal(ps, scales[perm])


def test_stochastic_prefix_matches_oracle(oracle, K, data):
    print("case fullsize absmax SR prefix", flush=True)
    dev = torch.device("cuda:0")
    _, dy = data
    seed, signs = 0x5EED_0123_4567, 0x0F0F_F0F0
    sv = np.array([-1 if (signs >> j) & 1 else 1 for j in range(32)])
    codes, scales, _, _ = K.quantize_mxfp4(dy.to(dev), 32, signs, K.QM_ABSMAX_SR, seed=seed, tiled=True)
    torch.cuda.synchronize()
    ref = oracle.quantize(to_oracle(dy[:64]), 32, signs=sv, mode=oracle.ABSMAX_SR, seed=seed)
    assert np.array_equal(to_oracle(K.untile_codes(codes)[:64]), ref["codes"])
    assert np.array_equal(to_oracle(scales[:64]), ref["scales"])


def test_transposed_and_requantize_column_slices(oracle, K, data):
    print("case fullsize transposed / requantize slices", flush=True)
    dev = torch.device("cuda:0")
    x, dy = data
    signs = 0xA5A5_5A5A
    sv = np.array([-1 if (signs >> j) & 1 else 1 for j in range(32)])
    # B4: logical [O, T] = dy^T; logical rows q0..q0+31 are columns q0..q0+31 of dy
    etc, ets, _, _ = K.quantize_mxfp4(dy.to(dev), 32, signs, K.QM_ABSMAX_RTN, transposed_in=True, tiled=True)
    etc = K.untile_codes(etc)
    torch.cuda.synchronize()
    for q0 in (0, 2048 + 32, O - 32):
        ref = oracle.quantize(to_oracle(dy[:, q0:q0 + 32].contiguous()), 32, signs=sv, mode=oracle.ABSMAX_RTN, transposed_in=True)
        assert np.array_equal(to_oracle(etc[q0:q0 + 32]), ref["codes"]), q0
        assert np.array_equal(to_oracle(ets[q0:q0 + 32]), ref["scales"]), q0
    # the random stream of the transposed tensor starts at logical offset 0: rows 0..31 also match with a seed
    seed = 77
    sc, ss, _, _ = K.quantize_mxfp4(dy.to(dev), 32, signs, K.QM_ABSMAX_SR, transposed_in=True, seed=seed)
    ref = oracle.quantize(to_oracle(dy[:, :32].contiguous()), 32, signs=sv, mode=oracle.ABSMAX_SR, transposed_in=True, seed=seed)
    assert np.array_equal(to_oracle(sc[:32]), ref["codes"]) and np.array_equal(to_oracle(ss[:32]), ref["scales"])
    # B5: re-quantize Q(x)^T; output rows c0..c0+31 come from the 32-column slice (one scale column) of Q(x)
    xc, xs, _, _ = K.quantize_mxfp4(x.to(dev), 32, None, K.QM_QUEST_RTN)
    xtc, xts, _ = K.requantize_transposed_mxfp4(K.tile_codes(xc), xs, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_RTN,
                                                tiled_in=True, tiled_out=True)
    xtc = K.untile_codes(xtc)
    torch.cuda.synchronize()
    for c0 in (0, 1024 + 64, I - 32):
        cs = to_oracle(xc[:, c0 // 2:(c0 + 32) // 2].contiguous())
        ss_ = to_oracle(xs[:, c0 // 32:c0 // 32 + 1].contiguous())
        ref = oracle.requantize_transposed(cs, ss_, post=1.0, val_dtype=oracle.BF16, hd=32, signs=sv, mode=oracle.ABSMAX_RTN)
        assert np.array_equal(to_oracle(xtc[c0:c0 + 32]), ref["codes"]), c0
        assert np.array_equal(to_oracle(xts[c0:c0 + 32]), ref["scales"]), c0


def test_gemm_rows_and_sample(oracle, K, data):
    print("case fullsize gemm 8192x4096x4096", flush=True)
    dev = torch.device("cuda:0")
    x, _ = data
    g = torch.Generator().manual_seed(9)
    w = (0.02 * torch.randn(O, I, generator=g)).to(torch.bfloat16)
    xc, xs, _, _ = K.quantize_mxfp4(x.to(dev), 32, None, K.QM_QUEST_RTN, tiled=True)
    wc, ws, _, _ = K.quantize_mxfp4(w.to(dev), 32, None, K.QM_QUEST_RTN, tiled=True)
    y = K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.float32, a_tiled=True, b_tiled=True)
    y16 = K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.bfloat16, a_tiled=True, b_tiled=True)
    assert torch.equal(y16, y.to(torch.bfloat16))
    # a 256-row panel alone (one tile row, same K order inside every tile): bitwise the same rows
    xr = K.untile_codes(xc)
    sub = K.gemm_mxfp4_tn(K.tile_codes(xr[4096:4352].contiguous()), xs[4096:4352].contiguous(), wc, ws, 1.0, torch.float32,
                          a_tiled=True, b_tiled=True, split_k=False)
    assert torch.equal(sub, y[4096:4352])
    # sampled rows against the float64 product of the de-quantized operands
    idx = torch.randint(0, T, (64,), generator=g)
    A = oracle.dequantize(to_oracle(xr[idx.to(dev)]), to_oracle(xs[idx.to(dev)])).astype(np.float64)
    B = oracle.dequantize(to_oracle(K.untile_codes(wc)), to_oracle(ws)).astype(np.float64)
    want = A @ B.T
    got = y[idx.to(dev)].cpu().numpy().astype(np.float64)
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel <= 1e-5, rel  # stated tolerance 1e-3


def test_linear_step_rows_against_oracle_pipeline(oracle, K, data):
    """Whole layer at full size: the first 64 token rows of y and of grad_x depend on those rows of x / dy and on W
    only, so the oracle pipeline on (x[:64], W, dy[:64]) with the same seeds must reproduce them."""
    print("case fullsize linear fwd+bwd", flush=True)
    import random
    import quartet_amd as q
    dev = torch.device("cuda:0")
    x, dy = data
    g = torch.Generator().manual_seed(11)
    w = (0.02 * torch.randn(O, I, generator=g)).to(torch.bfloat16)
    layer = q.QuantizedLinear(I, O, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
                              activation_quantizer=q.QuestMXFP4Quantizer(),
                              gradient_quantizer=q.AlbertTsengQuantizer(stochastic=True, rerotate=None),
                              backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(dev, torch.bfloat16)
    with torch.no_grad():
        layer.weight.copy_(w.to(dev))
    xd = x.to(dev).requires_grad_(True)
    random.seed(4242)
    y = layer(xd)
    y.backward(dy.to(dev))
    torch.cuda.synchronize()
    random.seed(4242)
    seeds = [random.getrandbits(63) for _ in range(4)]
    d = float(oracle.FOUR_THIRDS)
    n = 64
    qx = oracle.quantize(to_oracle(x[:n]), 32, mode=oracle.QUEST_RTN, want_mask=True)
    qw = oracle.quantize(to_oracle(w), 32, mode=oracle.QUEST_RTN)
    y_ref = oracle.gemm_tn(qx["codes"], qx["scales"], qw["codes"], qw["scales"])
    got = y[:n].detach().float().cpu().numpy().astype(np.float64)
    assert np.linalg.norm(got - y_ref) / np.linalg.norm(y_ref) < 4e-3  # bf16 output rounding
    qe = oracle.quantize(to_oracle(dy[:n]), 32, mode=oracle.ABSMAX_SR, seed=seeds[0])
    qwt = oracle.requantize_transposed(qw["codes"], qw["scales"], val_dtype=oracle.BF16, hd=32, mode=oracle.ABSMAX_SR, seed=seeds[1])
    gxq = oracle.gemm_tn(qe["codes"], qe["scales"], qwt["codes"], qwt["scales"], a_post=d, b_post=d)
    gxq16 = torch.from_numpy(gxq).to(torch.bfloat16)
    gx_ref = oracle.masked_hadamard_bwd(to_oracle(gxq16), 32, oracle.BF16, None, qx["mask"])
    gx_ref = torch.from_numpy(gx_ref.view(np.int16)).view(torch.bfloat16).float().numpy().astype(np.float64)
    gx = xd.grad[:n].float().cpu().numpy().astype(np.float64)
    assert np.linalg.norm(gx - gx_ref) / np.linalg.norm(gx_ref) < 1e-2  # two bf16 roundings on the way


def _signs_from_word(word):
    return np.array([-1 if (word >> j) & 1 else 1 for j in range(32)])


@pytest.mark.parametrize("rows,cols,dtype", [(32768, 1536, torch.float32), (8192, 4096, torch.bfloat16)])
def test_rmsnorm_quantize_sampled_rows_match_oracle(oracle, K, rows, cols, dtype):
    """The fused RMSNorm -> quantizer is row-local: sampled rows of a full-size result (the 800 M model's shape, and
    the benchmark layer's) must equal the oracle's result on those rows, factor included."""
    print(f"case fullsize rmsnorm_quantize rows={rows} cols={cols} {dtype}", flush=True)
    from quartet_amd import packed as P
    import quartet_amd as q
    dev = torch.device("cuda:0")
    gd = torch.Generator(device=dev).manual_seed(rows + cols)
    x = (3.0 * torch.randn(rows, cols, generator=gd, device=dev)).to(dtype)
    x[torch.rand(rows, cols, generator=gd, device=dev) < 1e-3] = 200.0
    gain = 1.0 + 0.1 * torch.randn(cols, generator=gd, device=dev)
    word = 0x6C1B93A5
    packed, factor = K.rmsnorm_quantize(x, gain, 1e-5, word, True)
    t = P.from_operand_buffer(packed, rows, cols, True, q.QuestMXFP4Quantizer()).to_layout("rowmajor")
    idx = torch.randint(0, rows, (96,), generator=torch.Generator().manual_seed(1))
    idx = torch.cat([idx, torch.tensor([0, rows - 1])])
    normed, want_factor = oracle.rmsnorm(to_oracle(x[idx.to(dev)]), gain.cpu().numpy(), 1e-5)
    want = oracle.quantize(normed, 32, signs=_signs_from_word(word), mode=oracle.QUEST_RTN, want_mask=True)
    assert np.array_equal(factor[idx.to(dev)].cpu().numpy().view(np.uint32), want_factor.view(np.uint32))
    assert np.array_equal(t.scales[idx.to(dev)].cpu().numpy(), want["scales"])
    assert np.array_equal(t.codes[idx.to(dev)].cpu().numpy(), want["codes"])
    assert np.array_equal(t.maskbits[idx.to(dev)].cpu().numpy(), want["mask"])


@pytest.mark.parametrize("rows,hidden", [(32768, 4096), (8192, 11008)])
def test_swiglu_quantize_sampled_rows_match_oracle(oracle, K, rows, hidden):
    print(f"case fullsize swiglu_quantize rows={rows} hidden={hidden}", flush=True)
    from quartet_amd import packed as P
    import quartet_amd as q
    dev = torch.device("cuda:0")
    gd = torch.Generator(device=dev).manual_seed(rows + hidden)
    h12 = (2.0 * torch.randn(rows, 2 * hidden, generator=gd, device=dev)).to(torch.bfloat16)
    word = 0x1F3D5B79
    packed = K.swiglu_quantize(h12, word, True)
    t = P.from_operand_buffer(packed, rows, hidden, True, q.QuestMXFP4Quantizer()).to_layout("rowmajor")
    idx = torch.randint(0, rows, (64,), generator=torch.Generator().manual_seed(2))
    idx = torch.cat([idx, torch.tensor([0, rows - 1])])
    prod = oracle.swiglu(to_oracle(h12[idx.to(dev)]))
    want = oracle.quantize(prod, 32, signs=_signs_from_word(word), mode=oracle.QUEST_RTN, want_mask=True)
    assert np.array_equal(t.scales[idx.to(dev)].cpu().numpy(), want["scales"])
    assert np.array_equal(t.codes[idx.to(dev)].cpu().numpy(), want["codes"])
    assert np.array_equal(t.maskbits[idx.to(dev)].cpu().numpy(), want["mask"])
