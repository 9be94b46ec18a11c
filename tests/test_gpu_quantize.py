"""GPU parity of the quantizer family against the CPU oracle: FP4 codes, E8M0 scales, clip-mask
bits and the de-quantized tensor must be bit-exact (integer/byte work), through the C ABI."""
import numpy as np
import pytest
import torch

from tests.util import make_input, sign_int, to_oracle

pytestmark = pytest.mark.gpu

MODES = {"quest_rtn": 0, "absmax_rtn": 1, "absmax_sr": 2, "quest_sr": 3}


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from quartet_amd import kernels
    return kernels


def _check(oracle, K, x, hd, mode, signs, transposed, u, seed, tag):
    dev = torch.device("cuda:0")
    sb = None if signs is None else sign_int(signs)
    want_mask = mode in (0, 3)
    codes, scales, mask, deq = K.quantize_mxfp4(x.to(dev), hd, sb, mode, transposed, None if u is None else u.to(dev),
                                                seed, want_mask=want_mask, want_dequant=True)
    torch.cuda.synchronize()
    ref = oracle.quantize(to_oracle(x), hd, signs=None if signs is None else signs.numpy(), mode=mode,
                          transposed_in=transposed, u=None if u is None else u.numpy(), seed=seed,
                          want_mask=want_mask, want_dequant=True)
    for name, got, want in (("scales", scales, ref["scales"]), ("codes", codes, ref["codes"]),
                            ("mask", mask, ref["mask"]), ("dequant", deq, ref["dequant"])):
        if want is None:
            continue
        g = to_oracle(got)
        if g.dtype == np.float32:
            g, want = g.view(np.uint32), want.view(np.uint32)
        bad = int((g != want).sum())
        assert bad == 0, f"{tag}: {name} differs in {bad} of {want.size} entries"


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("hd", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rowmajor_bit_exact(oracle, K, mode, hd, dtype):
    print(f"case rowmajor mode={mode} hd={hd} dtype={dtype}", flush=True)
    x = make_input(96, 1024, dtype, seed=hd + MODES[mode], zero_rows=2)
    g = torch.Generator().manual_seed(1)
    signs = torch.randint(0, 2, (hd,), generator=g) * 2 - 1
    u = torch.rand(x.shape, generator=g) if "sr" in mode else None
    _check(oracle, K, x, hd, MODES[mode], signs, False, u, 0, f"rowmajor/{mode}/{hd}/{dtype}")


@pytest.mark.parametrize("mode", ["absmax_sr", "quest_sr"])
@pytest.mark.parametrize("hd", [32, 128])
def test_philox_stream_bit_exact(oracle, K, mode, hd):
    print(f"case philox mode={mode} hd={hd}", flush=True)
    x = make_input(64, 512, torch.bfloat16, seed=3)
    _check(oracle, K, x, hd, MODES[mode], None, False, None, 0x1234_5678_9ABC, f"philox/{mode}/{hd}")


@pytest.mark.parametrize("mode", ["absmax_sr", "absmax_rtn", "quest_rtn"])
@pytest.mark.parametrize("hd", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_transposed_input_bit_exact(oracle, K, mode, hd, dtype):
    print(f"case transposed mode={mode} hd={hd} dtype={dtype}", flush=True)
    # physical [P=384, Q=200]: ragged against the 128x64 tile in both directions
    x = make_input(384, 200, dtype, seed=hd, zero_rows=1)
    g = torch.Generator().manual_seed(2)
    signs = torch.randint(0, 2, (hd,), generator=g) * 2 - 1
    u = torch.rand(200, 384, generator=g) if "sr" in mode else None
    _check(oracle, K, x, hd, MODES[mode], signs, True, u, 0, f"transposed/{mode}/{hd}/{dtype}")


@pytest.mark.parametrize("hd", [32, 64, 128])
@pytest.mark.parametrize("val_dtype", [torch.bfloat16, torch.float32])
def test_requantize_transposed_bit_exact(oracle, K, hd, val_dtype):
    print(f"case requant hd={hd} val_dtype={val_dtype}", flush=True)
    dev = torch.device("cuda:0")
    x = make_input(384, 160, torch.bfloat16, seed=5, zero_rows=1)
    q = oracle.quantize(to_oracle(x), 32, mode=oracle.QUEST_RTN)
    g = torch.Generator().manual_seed(3)
    signs = torch.randint(0, 2, (hd,), generator=g) * 2 - 1
    u = torch.rand(160, 384, generator=g)
    vd = oracle.BF16 if val_dtype == torch.bfloat16 else oracle.F32
    for mode, post in ((2, 1.0), (1, 1.0), (2, float(oracle.FOUR_THIRDS))):
        ref = oracle.requantize_transposed(q["codes"], q["scales"], post=post, val_dtype=vd, hd=hd,
                                           signs=signs.numpy(), mode=mode, u=u.numpy(), want_dequant=True)
        co, so, dq = K.requantize_transposed_mxfp4(torch.from_numpy(q["codes"]).to(dev),
                                                   torch.from_numpy(q["scales"]).to(dev), post, val_dtype, hd,
                                                   sign_int(signs), mode, u.to(dev), 0, want_dequant=True)
        torch.cuda.synchronize()
        assert np.array_equal(to_oracle(so), ref["scales"])
        assert np.array_equal(to_oracle(co), ref["codes"])
        a, b = to_oracle(dq), ref["dequant"]
        if a.dtype == np.float32:
            a, b = a.view(np.uint32), b.view(np.uint32)
        assert np.array_equal(a, b)


# The group-layout kernels serve Hadamard block 32 with round-to-nearest or the in-kernel Philox stream; these
# shapes meet their alignment rules (physical P % 128 == 0 for transposed input, R % 128 == 0 for the
# re-quantizer) with ragged and multi-tile extents in the other direction.
@pytest.mark.parametrize("mode", ["absmax_sr", "absmax_rtn", "quest_rtn", "quest_sr"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("P,Q", [(128, 32), (256, 200), (384, 320)])
def test_transposed_group_layout_bit_exact(oracle, K, mode, dtype, P, Q):
    print(f"case transposed-g32 mode={mode} dtype={dtype} P={P} Q={Q}", flush=True)
    x = make_input(P, Q, dtype, seed=P + Q, zero_rows=1)
    x[0:32, 5] = 0  # logical row 5 starts with an all-zero MX group
    g = torch.Generator().manual_seed(12)
    signs = torch.randint(0, 2, (32,), generator=g) * 2 - 1
    dev = torch.device("cuda:0")
    seed = 0x0BAD_5EED_0000_0001 + P
    codes, scales, _, deq = K.quantize_mxfp4(x.to(dev), 32, sign_int(signs), MODES[mode], True, None, seed,
                                             want_mask=False, want_dequant=True)
    torch.cuda.synchronize()
    ref = oracle.quantize(to_oracle(x), 32, signs=signs.numpy(), mode=MODES[mode], transposed_in=True, u=None,
                          seed=seed, want_mask=False, want_dequant=True)
    assert np.array_equal(to_oracle(scales), ref["scales"])
    assert np.array_equal(to_oracle(codes), ref["codes"])
    a, b = to_oracle(deq), ref["dequant"]
    if a.dtype == np.float32:
        a, b = a.view(np.uint32), b.view(np.uint32)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("mode", ["absmax_sr", "absmax_rtn"])
@pytest.mark.parametrize("val_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("R,C", [(128, 32), (256, 160), (384, 512)])
def test_requantize_group_layout_bit_exact(oracle, K, mode, val_dtype, R, C):
    print(f"case requant-g32 mode={mode} val_dtype={val_dtype} R={R} C={C}", flush=True)
    dev = torch.device("cuda:0")
    x = make_input(R, C, torch.bfloat16, seed=R + C, zero_rows=1)
    q = oracle.quantize(to_oracle(x), 32, mode=oracle.QUEST_RTN)
    g = torch.Generator().manual_seed(13)
    signs = torch.randint(0, 2, (32,), generator=g) * 2 - 1
    vd = oracle.BF16 if val_dtype == torch.bfloat16 else oracle.F32
    seed = 0x7777_0000_1234 + C
    for post in (1.0, float(oracle.FOUR_THIRDS)):
        ref = oracle.requantize_transposed(q["codes"], q["scales"], post=post, val_dtype=vd, hd=32, signs=signs.numpy(),
                                           mode=MODES[mode], u=None, seed=seed, want_dequant=True)
        co, so, dq = K.requantize_transposed_mxfp4(torch.from_numpy(q["codes"]).to(dev),
                                                   torch.from_numpy(q["scales"]).to(dev), post, val_dtype, 32,
                                                   sign_int(signs), MODES[mode], None, seed, want_dequant=True)
        torch.cuda.synchronize()
        assert np.array_equal(to_oracle(so), ref["scales"])
        assert np.array_equal(to_oracle(co), ref["codes"])
        a, b = to_oracle(dq), ref["dequant"]
        if a.dtype == np.float32:
            a, b = a.view(np.uint32), b.view(np.uint32)
        assert np.array_equal(a, b)


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("hd", [32, 64, 128])
def test_rowmajor_group_layout_seeded(oracle, K, mode, dtype, hd):
    print(f"case rowmajor-group mode={mode} dtype={dtype} hd={hd}", flush=True)
    # 33 rows x 2176 columns: the element count is not a multiple of the kernel's per-block share
    x = make_input(33, 2176, dtype, seed=21 + hd, zero_rows=1)
    g = torch.Generator().manual_seed(14 + hd)
    signs = torch.randint(0, 2, (hd,), generator=g) * 2 - 1
    _check(oracle, K, x, hd, MODES[mode], signs, False, None, 0xFEED_F00D_CAFE + hd, f"rowmajor-group/{mode}/{dtype}/{hd}")


@pytest.mark.parametrize("mode", ["absmax_rtn", "absmax_sr"])
@pytest.mark.parametrize("transposed", [False, True])
def test_tiny_magnitudes_follow_the_definition(oracle, K, mode, transposed):
    """Groups whose maximum lies far below the normal range (down into the denormals) and tiny elements inside
    ordinary groups: the quotient by fl32(4/3) is computed from the scaled value, as the definition says."""
    print(f"case tiny magnitudes mode={mode} transposed={transposed}", flush=True)
    g = torch.Generator().manual_seed(77)
    x = torch.randn(128, 256, generator=g)
    exps = torch.tensor([0, -20, -50, -59, -60, -61, -70, -90, -100, -104, -110, -120, -124, -126, -130, -140])
    x = x * torch.pow(2.0, exps.repeat_interleave(8).double())[:, None].float()   # row r scaled by 2^exps[r // 8]
    x[::8, ::5] *= 2.0 ** -40                                                       # much smaller elements inside each group
    x[3, :32] = torch.tensor([2.0 ** -149, -(2.0 ** -149), 2.0 ** -148, 0.0] * 8)   # smallest denormals and zero
    if transposed:
        x = x.t().contiguous()
    signs = torch.randint(0, 2, (32,), generator=g) * 2 - 1
    _check(oracle, K, x, 32, MODES[mode], signs, transposed, None, 0xBEEF + int(transposed), f"tiny/{mode}/{transposed}")


@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_already_rotated_input_passes_through(oracle, K, mode, dtype):
    """hadamard_dim 1: the groups of 32 are quantized as they are (the caller applied a dense rotation)."""
    print(f"case pass-through mode={mode} dtype={dtype}", flush=True)
    x = make_input(40, 384, dtype, seed=31, zero_rows=1)
    _check(oracle, K, x, 1, MODES[mode], None, False, None, 0xABCDEF + MODES[mode], f"pass-through/{mode}/{dtype}")


def test_pass_through_rejections(K):
    from quartet_amd._lib import QuartetHipError
    dev = torch.device("cuda:0")
    x = torch.zeros(32, 128, dtype=torch.bfloat16, device=dev)
    u = torch.rand(32, 128, device=dev)
    for kwargs in (dict(transposed_in=True), dict(u=u, mode=K.QM_ABSMAX_SR), dict(sign_bits=5), dict(tiled=True)):
        with pytest.raises(QuartetHipError, match="hadamard_dim 1"):
            K.quantize_mxfp4(x, 1, **{"sign_bits": None, "mode": K.QM_QUEST_RTN, **kwargs})
    with pytest.raises(QuartetHipError):
        K.requantize_transposed_mxfp4(torch.zeros(32, 64, dtype=torch.uint8, device=dev),
                                      torch.zeros(32, 4, dtype=torch.uint8, device=dev), hadamard_dim=1)


# Tiled code layout ([R/16][C/128][16][64 bytes]): the same bytes as the row-major codes, permuted; scales, mask
# and the de-quantized tensor are unaffected.
@pytest.mark.parametrize("mode", list(MODES))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("R,C", [(16, 128), (48, 640), (256, 1024)])
def test_rowmajor_tiled_codes(oracle, K, mode, dtype, R, C):
    print(f"case rowmajor-tiled mode={mode} dtype={dtype} R={R} C={C}", flush=True)
    dev = torch.device("cuda:0")
    x = make_input(R, C, dtype, seed=R + C, zero_rows=1)
    g = torch.Generator().manual_seed(15)
    signs = torch.randint(0, 2, (32,), generator=g) * 2 - 1
    seed = 0x1111_2222_3333 + R
    want_mask = "quest" in mode
    codes, scales, mask, deq = K.quantize_mxfp4(x.to(dev), 32, sign_int(signs), MODES[mode], False, None, seed,
                                                want_mask=want_mask, want_dequant=True, tiled=True)
    plain = K.quantize_mxfp4(x.to(dev), 32, sign_int(signs), MODES[mode], False, None, seed, want_mask=want_mask)
    torch.cuda.synchronize()
    ref = oracle.quantize(to_oracle(x), 32, signs=signs.numpy(), mode=MODES[mode], seed=seed, want_mask=want_mask,
                          want_dequant=True)
    assert np.array_equal(to_oracle(K.untile_codes(codes)), ref["codes"])
    assert torch.equal(K.tile_codes(plain[0]), codes)
    assert np.array_equal(to_oracle(scales), ref["scales"])
    if want_mask:
        assert np.array_equal(to_oracle(mask), ref["mask"])
    a, b = to_oracle(deq), ref["dequant"]
    assert np.array_equal(a.view(np.uint32) if a.dtype == np.float32 else a, b.view(np.uint32) if b.dtype == np.float32 else b)


@pytest.mark.parametrize("mode", ["absmax_sr", "absmax_rtn"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("P,Q", [(128, 16), (256, 208), (384, 320)])
def test_transposed_tiled_codes(oracle, K, mode, dtype, P, Q):
    print(f"case transposed-tiled mode={mode} dtype={dtype} P={P} Q={Q}", flush=True)
    dev = torch.device("cuda:0")
    x = make_input(P, Q, dtype, seed=P + Q)
    seed = 0x4444_5555 + Q
    codes, scales, _, _ = K.quantize_mxfp4(x.to(dev), 32, 0x0F0F00FF, MODES[mode], True, None, seed, tiled=True)
    torch.cuda.synchronize()
    signs = np.array([-1 if (0x0F0F00FF >> j) & 1 else 1 for j in range(32)])
    ref = oracle.quantize(to_oracle(x), 32, signs=signs, mode=MODES[mode], transposed_in=True, seed=seed)
    assert np.array_equal(to_oracle(K.untile_codes(codes)), ref["codes"])
    assert np.array_equal(to_oracle(scales), ref["scales"])


@pytest.mark.parametrize("tiled_in,tiled_out", [(True, True), (True, False), (False, True)])
@pytest.mark.parametrize("R,C", [(128, 128), (256, 384), (384, 1024)])
def test_requantize_tiled_codes(oracle, K, tiled_in, tiled_out, R, C):
    print(f"case requant-tiled in={tiled_in} out={tiled_out} R={R} C={C}", flush=True)
    dev = torch.device("cuda:0")
    x = make_input(R, C, torch.bfloat16, seed=R + C)
    q = oracle.quantize(to_oracle(x), 32, mode=oracle.QUEST_RTN)
    seed = 0x6666 + C
    ref = oracle.requantize_transposed(q["codes"], q["scales"], post=1.0, val_dtype=oracle.BF16, hd=32, signs=None,
                                       mode=oracle.ABSMAX_SR, u=None, seed=seed)
    cin = torch.from_numpy(q["codes"]).to(dev)
    if tiled_in:
        cin = K.tile_codes(cin)
    co, so, _ = K.requantize_transposed_mxfp4(cin, torch.from_numpy(q["scales"]).to(dev), 1.0, torch.bfloat16, 32, None,
                                              K.QM_ABSMAX_SR, None, seed, tiled_in=tiled_in, tiled_out=tiled_out)
    torch.cuda.synchronize()
    if tiled_out:
        co = K.untile_codes(co)
    assert np.array_equal(to_oracle(co), ref["codes"])
    assert np.array_equal(to_oracle(so), ref["scales"])


def test_tiled_layout_rejections(K):
    from quartet_amd._lib import QuartetHipError
    dev = torch.device("cuda:0")
    x = torch.randn(24, 128, device=dev).to(torch.bfloat16)       # 24 rows: not a multiple of 16
    with pytest.raises(QuartetHipError):
        K.quantize_mxfp4(x, 32, None, 0, tiled=True)
    x = torch.randn(32, 256, device=dev).to(torch.bfloat16)
    with pytest.raises(QuartetHipError):                          # tiled codes exist for Hadamard block 32 only
        K.quantize_mxfp4(x, 64, None, 0, tiled=True)
    with pytest.raises(QuartetHipError):                          # and not with explicit uniforms
        K.quantize_mxfp4(x, 32, None, 2, u=torch.rand(32, 256, device=dev), tiled=True)
    c = torch.zeros(128, 64, dtype=torch.uint8, device=dev)
    sc = torch.full((128, 4), 127, dtype=torch.uint8, device=dev)
    with pytest.raises(QuartetHipError):                          # GEMM: 128 rows are less than one 256-row tile
        K.gemm_mxfp4_tn(c, sc, c, sc, 1.0, torch.float32, a_tiled=True)


def test_order_independent_integer_fixture(oracle, K):
    # x = S @ g with small integers and hd = 64: every partial sum is exact, so the expected
    # rotated values (8*g) and hence codes/scales do not depend on any summation order.
    import scipy.linalg
    rng = np.random.default_rng(0)
    g = rng.integers(-3, 4, size=(32, 64)).astype(np.float64)
    x = torch.from_numpy((g @ scipy.linalg.hadamard(64)).astype(np.float32))
    for mode in (0, 1):
        _check(oracle, K, x, 64, mode, None, False, None, 0, f"integer/{mode}")
        _check(oracle, K, x.to(torch.bfloat16), 64, mode, None, False, None, 0, f"integer-bf16/{mode}")


def test_dequantize_and_hadamard_bwd(oracle, K):
    dev = torch.device("cuda:0")
    x = make_input(64, 512, torch.bfloat16, seed=9)
    for mode, post in ((0, 1.0), (1, float(oracle.FOUR_THIRDS))):
        q = oracle.quantize(to_oracle(x), 32, mode=mode, want_mask=True)
        for od, oc in ((torch.float32, oracle.F32), (torch.bfloat16, oracle.BF16)):
            got = K.dequantize_mxfp4(torch.from_numpy(q["codes"]).to(dev), torch.from_numpy(q["scales"]).to(dev), post, od)
            want = oracle.dequantize(q["codes"], q["scales"], post, oc)
            a = to_oracle(got)
            assert np.array_equal(a.view(np.uint32) if a.dtype == np.float32 else a,
                                  want.view(np.uint32) if want.dtype == np.float32 else want)
    gen = torch.Generator().manual_seed(4)
    for hd in (32, 64, 128):
        signs = torch.randint(0, 2, (hd,), generator=gen) * 2 - 1
        maskbits = torch.randint(0, 256, (64, 512 // 8), generator=gen, dtype=torch.uint8)
        for gd, od in ((torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32), (torch.bfloat16, torch.float32)):
            g = make_input(64, 512, gd, seed=hd)
            for mb in (maskbits, None):
                got = K.masked_hadamard_bwd(g.to(dev), hd, torch.bfloat16, sign_int(signs), None if mb is None else mb.to(dev), od)
                want = oracle.masked_hadamard_bwd(to_oracle(g), hd, oracle.BF16, signs.numpy(),
                                                  None if mb is None else mb.numpy(),
                                                  oracle.BF16 if od == torch.bfloat16 else oracle.F32)
                a = to_oracle(got)
                assert np.array_equal(a.view(np.uint32) if a.dtype == np.float32 else a,
                                      want.view(np.uint32) if want.dtype == np.float32 else want), (hd, gd, od)


def test_empty_and_rejected_inputs(K):
    dev = torch.device("cuda:0")
    from quartet_amd._lib import QuartetHipError
    c, s, m, d = K.quantize_mxfp4(torch.empty(0, 64, dtype=torch.bfloat16, device=dev), want_mask=True, want_dequant=True)
    assert c.shape == (0, 32) and s.shape == (0, 2)
    with pytest.raises(QuartetHipError, match="multiple of hadamard_dim"):
        K.quantize_mxfp4(torch.zeros(4, 48, dtype=torch.bfloat16, device=dev))
    with pytest.raises(QuartetHipError, match="hadamard_dim"):
        K.quantize_mxfp4(torch.zeros(4, 64, dtype=torch.bfloat16, device=dev), hadamard_dim=16)
    with pytest.raises(QuartetHipError):
        K.quantize_mxfp4(torch.zeros(4, 64, dtype=torch.bfloat16))  # CPU tensor: no fallback


def _orthogonal(seed):
    """A dense 32 x 32 rotation as re_randomize("O32") draws it: U V^T of a Gaussian matrix's SVD."""
    g = torch.Generator().manual_seed(seed)
    u, _, vh = torch.linalg.svd(torch.randn(32, 32, generator=g))
    return (u @ vh).contiguous()


def _same_bits(got, want, tag):
    for name in ("scales", "codes", "mask", "dequant"):
        if want.get(name) is None or got.get(name) is None:
            continue
        g, w = to_oracle(got[name]), want[name]
        if g.dtype == np.float32:
            g, w = g.view(np.uint32), w.view(np.uint32)
        bad = int((g != w).sum())
        assert bad == 0, f"{tag}: {name} differs in {bad} of {w.size} entries"


@pytest.mark.parametrize("mode", ["quest_rtn", "absmax_rtn", "absmax_sr"])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_dense_rotation_kernels_bit_exact(oracle, K, mode, dtype):
    """rerotate="O32": every group of 32 is multiplied by a dense 32 x 32 matrix on the matrix pipe (one fused
    multiply-add per term, ascending k) and quantized.  Codes, scales, mask bits and de-quantized values must equal
    the oracle's bit for bit: row-major input (ragged and tiled shapes), transposed input, and the transposing
    re-quantizer of a packed tensor, with the in-kernel random stream for stochastic rounding."""
    print(f"case dense rotation mode={mode} dtype={dtype}", flush=True)
    dev = torch.device("cuda:0")
    H = _orthogonal(17)
    m = MODES[mode]
    want_mask = mode == "quest_rtn"
    seed = 0xABCD_1234_5678 if "sr" in mode else 0
    odt = oracle.BF16 if dtype == torch.bfloat16 else oracle.F32
    for rows, cols, tiled in ((100, 96, False), (272, 640, False), (128, 256, True)):
        x = make_input(rows, cols, dtype, seed=rows + cols, zero_rows=1)
        codes, scales, mask, deq = K.quantize_mxfp4_dense(x.to(dev), H.to(dev), m, seed=seed, want_mask=want_mask, want_dequant=True,
                                                          tiled=tiled)
        ref = oracle.quantize(to_oracle(x), mode=m, seed=seed, want_mask=want_mask, want_dequant=True, matrix=H.numpy())
        _same_bits(dict(scales=scales, codes=K.untile_codes(codes) if tiled else codes, mask=mask, dequant=deq), ref,
                   f"dense rowmajor {rows}x{cols} tiled={tiled}")
    if mode != "quest_rtn":   # the transposing kernels serve the gradient quantizer: no clip mask
        for p, q_, tiled in ((256, 72, False), (128, 200, False), (256, 80, True)):
            x = make_input(p, q_, dtype, seed=p + q_)   # physical [P, Q]; logical [Q, P]
            codes, scales, _, deq = K.quantize_mxfp4_dense(x.to(dev), H.to(dev), m, transposed_in=True, seed=seed, want_dequant=True,
                                                           tiled=tiled)
            ref = oracle.quantize(to_oracle(x), mode=m, seed=seed, transposed_in=True, want_dequant=True, matrix=H.numpy())
            _same_bits(dict(scales=scales, codes=K.untile_codes(codes) if tiled else codes, dequant=deq), ref,
                       f"dense transposed {p}x{q_} tiled={tiled}")
        for R, C, tiled in ((256, 96, False), (640, 160, False), (512, 256, True), (1152, 128, True)):
            src = make_input(R, C, torch.bfloat16, seed=R + C)
            qc = oracle.quantize(to_oracle(src), 32, mode=oracle.QUEST_RTN)
            cin = torch.from_numpy(qc["codes"]).to(dev)
            sin = torch.from_numpy(qc["scales"]).to(dev)
            codes, scales, deq = K.requantize_transposed_mxfp4_dense(K.tile_codes(cin) if tiled else cin, sin, H.to(dev), 1.0, dtype, m,
                                                                     seed=seed, want_dequant=True, tiled_in=tiled, tiled_out=tiled)
            ref = oracle.requantize_transposed(qc["codes"], qc["scales"], 1.0, odt, mode=m, seed=seed, want_dequant=True,
                                               matrix=H.numpy())
            _same_bits(dict(scales=scales, codes=K.untile_codes(codes) if tiled else codes, dequant=deq), ref,
                       f"dense requantize {R}x{C} tiled={tiled}")


def test_dense_rotation_with_the_hadamard_matrix_is_close_to_the_butterfly(oracle, K):
    """The Hadamard matrix handed over as a dense matrix: same scales, and codes that differ only where the two
    summation orders round a rotated value differently."""
    dev = torch.device("cuda:0")
    x = make_input(256, 512, torch.bfloat16, seed=5)
    c = float(oracle.hadamard_scale(32, oracle.BF16))
    Hd = torch.from_numpy(oracle.sylvester(32).astype(np.float32) * np.float32(c))
    a = K.quantize_mxfp4(x.to(dev), 32, None, K.QM_QUEST_RTN, want_mask=True)
    b = K.quantize_mxfp4_dense(x.to(dev), Hd.to(dev), K.QM_QUEST_RTN, want_mask=True)
    assert torch.equal(a[1], b[1])
    assert float((a[0] != b[0]).float().mean()) < 0.01
