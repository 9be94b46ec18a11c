"""Parity at the benchmark's full sizes (tokens 8192, in 4096, out 4096 and 11008; the quantizer on [rows x 4096] for
rows 4096, 16384 and 65536 with Hadamard blocks 32, 64 and 128), where the CPU oracle cannot process whole tensors in
test time.  Each check is a size-independent property that reduces
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
OUTS = [4096, 11008]   # the two out-feature counts of the isolated-layer configuration


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from quartet_amd import kernels
    return kernels


def _make_data(out_features):
    g = torch.Generator().manual_seed(123)
    x = torch.randn(T, I, generator=g)
    heavy = torch.rand(T, I, generator=g) < 0.01
    x = torch.where(heavy, 30.0 * torch.randn(T, I, generator=g), x).to(torch.bfloat16)
    dy = (1e-3 * torch.randn(T, out_features, generator=g)).to(torch.bfloat16)
    return x, dy


@pytest.fixture(scope="module")
def data():
    return _make_data(O)


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


C4_ROWS = [4096, 16384, 65536]   # 16 Mi, 64 Mi and 256 Mi elements as [rows x 4096]


@pytest.mark.parametrize("rows", C4_ROWS)
@pytest.mark.parametrize("hd", [32, 64, 128])
@pytest.mark.parametrize("mode", ["quest_rtn_mask", "absmax_rtn", "absmax_sr"])
def test_quantizer_sweep_sampled_rows_match_oracle(oracle, K, rows, hd, mode):
    """The quantizer-only configuration at its real sizes: Gaussian data with 0.1 % entries at +-1e3, three modes,
    Hadamard blocks 32 / 64 / 128.  A Hadamard block never crosses a row, so sampled rows of the big result must equal
    the oracle's result on those rows; with stochastic rounding the in-kernel stream is keyed by the flat element
    offset, so the oracle is fed the stream's uniforms at the sampled rows' offsets."""
    print(f"case quantizer sweep rows={rows} hd={hd} {mode}", flush=True)
    dev = torch.device("cuda:0")
    cols = 4096
    seed = 1000 * hd + rows
    gd = torch.Generator(device=dev).manual_seed(seed)
    xd = torch.randn(rows, cols, generator=gd, device=dev)
    spike = torch.rand(rows, cols, generator=gd, device=dev) < 1e-3
    sgn = torch.where(torch.rand(rows, cols, generator=gd, device=dev) < 0.5, -1e3, 1e3)
    xd = torch.where(spike, sgn, xd).to(torch.bfloat16)
    signs = (0x9D2C5681 | (0x3A5F01C7 << 32) | (0xC0FFEE11 << 64) | (0x13579BDF << 96)) & ((1 << hd) - 1)
    sv = np.array([-1 if (signs >> j) & 1 else 1 for j in range(hd)])
    qmode = {"quest_rtn_mask": K.QM_QUEST_RTN, "absmax_rtn": K.QM_ABSMAX_RTN, "absmax_sr": K.QM_ABSMAX_SR}[mode]
    omode = {"quest_rtn_mask": oracle.QUEST_RTN, "absmax_rtn": oracle.ABSMAX_RTN, "absmax_sr": oracle.ABSMAX_SR}[mode]
    want_mask = mode == "quest_rtn_mask"
    kseed = 0xC0DE_0000 + rows + hd
    codes, scales, mask, _ = K.quantize_mxfp4(xd, hd, signs, qmode, want_mask=want_mask, seed=kseed)
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(seed)
    idx = torch.cat([torch.arange(0, 8), torch.randint(0, rows, (80,), generator=g), torch.arange(rows - 8, rows)])
    u = None
    if mode == "absmax_sr":
        offsets = idx.numpy().astype(np.int64)[:, None] * cols + np.arange(cols, dtype=np.int64)[None, :]
        u = oracle.philox_uniform_at(kseed, offsets)
    ref = oracle.quantize(to_oracle(xd[idx.to(dev)]), hd, signs=sv, mode=omode, want_mask=want_mask, u=u)
    assert np.array_equal(_rows(scales, idx.to(dev)), ref["scales"])
    assert np.array_equal(_rows(codes, idx.to(dev)), ref["codes"])
    if want_mask:
        assert np.array_equal(_rows(mask, idx.to(dev)), ref["mask"])
    if hd == 32:   # the tiled code layout (Hadamard block 32 only) holds the same bytes
        tcodes, tscales, tmask, _ = K.quantize_mxfp4(xd, hd, signs, qmode, want_mask=want_mask, seed=kseed, tiled=True)
        assert torch.equal(K.untile_codes(tcodes), codes) and torch.equal(tscales, scales)
        assert not want_mask or torch.equal(tmask, mask)


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


def _random_operand(K, rows, cols, seed, mode, dev, tiled=True):
    """A packed [rows, cols] operand (tiled codes unless told otherwise) quantized from seeded Gaussian data generated on
    the GPU."""
    gd = torch.Generator(device=dev).manual_seed(seed)
    t = torch.randn(rows, cols, generator=gd, device=dev).to(torch.bfloat16)
    codes, scales, _, _ = K.quantize_mxfp4(t, 32, None, mode, tiled=tiled, seed=seed)
    return codes, scales


# the three products of the isolated layer at out = 4096 and out = 11008 (forward, grad-input, grad-weight: M x N x K)
GEMM_SHAPES = [(T, 4096, I), (4096, I, T), (T, 11008, I), (T, I, 11008), (11008, I, T)]
# forward / grad-input products of the two Llama configurations (32768 tokens): short contractions on the 256 x 128
# kernel (K = 640, with N = 1728 hanging over a tile edge; K = 1728 = 13.5 steps of 128 closes with a half step), K = 1536 and
# 1920 on the persistent one
GEMM_SHAPES += [(32768, 3456, 640), (32768, 1728, 640), (32768, 640, 1728), (32768, 4608, 1536), (32768, 640, 1920)]


@pytest.mark.parametrize("M,N,Kdim", GEMM_SHAPES)
def test_gemm_rows_and_sample(oracle, K, M, N, Kdim):
    print(f"case fullsize gemm {M}x{N}x{Kdim}", flush=True)
    from quartet_amd import _lib
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(9)
    # forward-like operands for the token-major products, absmax-coded ones (whole E2M1 range, post-scale 4/3) for the
    # weight-gradient shape
    absmax = Kdim == T
    mode = K.QM_ABSMAX_RTN if absmax else K.QM_QUEST_RTN
    post = float(oracle.FOUR_THIRDS) if absmax else 1.0
    tl = Kdim % 128 == 0 and N % 128 == 0    # what the tiled layout needs
    ac, as_ = _random_operand(K, M, Kdim, 100 + M, mode, dev, tl)
    bc, bs = _random_operand(K, N, Kdim, 200 + N, mode, dev, tl)
    alpha = post * post
    y = K.gemm_mxfp4_tn(ac, as_, bc, bs, alpha, torch.float32, a_tiled=tl, b_tiled=tl)
    y16 = K.gemm_mxfp4_tn(ac, as_, bc, bs, alpha, torch.bfloat16, a_tiled=tl, b_tiled=tl)
    assert torch.equal(y16, y.to(torch.bfloat16))
    ar = K.untile_codes(ac) if tl else ac
    if _lib.lib().qm_gemm_workspace_bytes(M, N, Kdim) == 0:
        # a 256-row panel alone (one tile row, same K order inside every tile): bitwise the same rows
        r0 = (M // 2 // 256) * 256
        a_sub = ar[r0:r0 + 256].contiguous()
        sub = K.gemm_mxfp4_tn(K.tile_codes(a_sub) if tl else a_sub, as_[r0:r0 + 256].contiguous(), bc, bs, alpha,
                              torch.float32, a_tiled=tl, b_tiled=tl, split_k=False)
        assert torch.equal(sub, y[r0:r0 + 256])
    # sampled rows (first, last and random ones) against the float64 product of the de-quantized operands
    idx = torch.cat([torch.tensor([0, M - 1]), torch.randint(0, M, (46,), generator=g)]).to(dev)
    A = oracle.dequantize(to_oracle(ar[idx]), to_oracle(as_[idx]), post).astype(np.float64)
    B = oracle.dequantize(to_oracle(K.untile_codes(bc) if tl else bc), to_oracle(bs), post).astype(np.float64)
    want = A @ B.T
    got = y[idx].cpu().numpy().astype(np.float64)
    rel = np.linalg.norm(got - want) / np.linalg.norm(want)
    assert rel <= 1e-5, rel  # stated tolerance 1e-3


@pytest.mark.parametrize("out_features", OUTS)
def test_linear_step_rows_against_oracle_pipeline(oracle, K, out_features):
    """Whole layer at full size.  The first 64 token rows of y and of grad_x depend on those rows of x / dy and on W
    only, and the first 32 rows of grad_W on the first 32 columns of dy and on all of x: the oracle pipeline on those
    slices with the same seeds must reproduce them (the random streams are keyed by flat offsets, which agree for a
    prefix of rows)."""
    print(f"case fullsize linear fwd+bwd out={out_features}", flush=True)
    import random
    import quartet_amd as q
    dev = torch.device("cuda:0")
    Of = out_features
    x, dy = _make_data(Of)
    g = torch.Generator().manual_seed(11)
    w = (0.02 * torch.randn(Of, I, generator=g)).to(torch.bfloat16)
    layer = q.QuantizedLinear(I, Of, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
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
    qx = oracle.quantize(to_oracle(x), 32, mode=oracle.QUEST_RTN, want_mask=True)
    qw = oracle.quantize(to_oracle(w), 32, mode=oracle.QUEST_RTN, want_mask=True)
    y_ref = oracle.gemm_tn(qx["codes"][:n], qx["scales"][:n], qw["codes"], qw["scales"])
    got = y[:n].detach().float().cpu().numpy().astype(np.float64)
    assert np.linalg.norm(got - y_ref) / np.linalg.norm(y_ref) < 4e-3  # bf16 output rounding

    def bf16_round(a):
        return to_oracle(torch.from_numpy(a).to(torch.bfloat16))

    def as_f64(bits):
        return torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).float().numpy().astype(np.float64)
    # grad_x: B1, B2, B3, B7
    qe = oracle.quantize(to_oracle(dy[:n]), 32, mode=oracle.ABSMAX_SR, seed=seeds[0])
    qwt = oracle.requantize_transposed(qw["codes"], qw["scales"], val_dtype=oracle.BF16, hd=32, mode=oracle.ABSMAX_SR, seed=seeds[1])
    gxq = oracle.gemm_tn(qe["codes"], qe["scales"], qwt["codes"], qwt["scales"], a_post=d, b_post=d)
    gx_ref = as_f64(oracle.masked_hadamard_bwd(bf16_round(gxq), 32, oracle.BF16, None, qx["mask"][:n]))
    gx = xd.grad[:n].float().cpu().numpy().astype(np.float64)
    assert np.linalg.norm(gx - gx_ref) / np.linalg.norm(gx_ref) < 1e-2  # two bf16 roundings on the way
    # grad_W: B4, B5, B6, B8 (contraction over all 8192 tokens)
    m = 32
    qet = oracle.quantize(to_oracle(dy[:, :m].contiguous()), 32, mode=oracle.ABSMAX_SR, transposed_in=True, seed=seeds[2])
    qxt = oracle.requantize_transposed(qx["codes"], qx["scales"], val_dtype=oracle.BF16, hd=32, mode=oracle.ABSMAX_SR, seed=seeds[3])
    gwq = oracle.gemm_tn(qet["codes"], qet["scales"], qxt["codes"], qxt["scales"], a_post=d, b_post=d)
    gw_ref = as_f64(oracle.masked_hadamard_bwd(bf16_round(gwq), 32, oracle.BF16, None, qw["mask"][:m]))
    gw = layer.weight.grad[:m].float().cpu().numpy().astype(np.float64)
    assert np.linalg.norm(gw - gw_ref) / np.linalg.norm(gw_ref) < 1e-2


@pytest.mark.parametrize("out_features", OUTS)
@pytest.mark.parametrize("rerotate", [None, "signs"])
def test_linear_step_equals_the_composition_of_its_kernels(K, out_features, rerotate):
    """End to end at full size, bit for bit: the layer's y, grad_x and grad_W equal what the same kernels give when they
    are called one by one through their own entry points with the layer's sign flips and seeds (two forward quantizers,
    the product; two gradient quantizers, two re-quantizers, and the two products with the inverse rotation in their
    epilogue).  Each of those entry points is checked against the oracle on its own, at full size on sampled rows and
    exhaustively at small sizes, so every element of the layer's results is tied to the oracle through them."""
    print(f"case fullsize linear step against its kernels out={out_features} rerotate={rerotate}", flush=True)
    import random
    import quartet_amd as q
    dev = torch.device("cuda:0")
    Of = out_features
    x, dy = _make_data(Of)
    g = torch.Generator().manual_seed(11)
    w = (0.02 * torch.randn(Of, I, generator=g)).to(torch.bfloat16)
    layer = q.QuantizedLinear(I, Of, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
                              activation_quantizer=q.QuestMXFP4Quantizer(),
                              gradient_quantizer=q.AlbertTsengQuantizer(stochastic=True, rerotate=rerotate),
                              backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(dev, torch.bfloat16)
    with torch.no_grad():
        layer.weight.copy_(w.to(dev))
    xd = x.to(dev).requires_grad_(True)
    torch.manual_seed(77)      # the sign flips of re_randomize
    random.seed(4242)          # the four stochastic-rounding seeds
    y = layer(xd)
    y.backward(dy.to(dev))
    torch.cuda.synchronize()
    random.seed(4242)
    seeds = [random.getrandbits(63) for _ in range(4)]
    signs = layer.backward_scheme.g_quantizer.sign_bits or None
    assert (signs is not None) == (rerotate == "signs")
    tl = True
    alpha = float(torch.tensor(K.FOUR_THIRDS, dtype=torch.float32) * torch.tensor(K.FOUR_THIRDS, dtype=torch.float32))
    xq, wq, e = x.to(dev), w.to(dev), dy.to(dev)
    xc, xs, xm, _ = K.quantize_mxfp4(xq, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)
    wc, ws, wm, _ = K.quantize_mxfp4(wq, 32, None, K.QM_QUEST_RTN, want_mask=True, tiled=tl)
    assert torch.equal(y.detach(), K.gemm_mxfp4_tn(xc, xs, wc, ws, 1.0, torch.bfloat16, a_tiled=tl, b_tiled=tl))
    ec, es, _, _ = K.quantize_mxfp4(e, 32, signs, K.QM_ABSMAX_SR, seed=seeds[0], tiled=tl)
    wtc, wts, _ = K.requantize_transposed_mxfp4(wc, ws, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=seeds[1], tiled_in=tl, tiled_out=tl)
    etc, ets, _, _ = K.quantize_mxfp4(e, 32, signs, K.QM_ABSMAX_SR, transposed_in=True, seed=seeds[2], tiled=tl)
    xtc, xts, _ = K.requantize_transposed_mxfp4(xc, xs, 1.0, torch.bfloat16, 32, signs, K.QM_ABSMAX_SR, seed=seeds[3], tiled_in=tl, tiled_out=tl)
    assert K.gemm_fuses_rotation(es, wts, T, I, Of) and K.gemm_fuses_rotation(ets, xts, Of, I, T)
    gx = K.gemm_mxfp4_tn_rotated(ec, es, wtc, wts, xm, alpha, torch.bfloat16, None, a_tiled=tl, b_tiled=tl)
    gw = K.gemm_mxfp4_tn_rotated(etc, ets, xtc, xts, wm, alpha, torch.bfloat16, None, a_tiled=tl, b_tiled=tl)
    assert torch.equal(xd.grad, gx)
    assert torch.equal(layer.weight.grad, gw)


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
