"""GPU parity of the MXFP4 x MXFP4 GEMM against the oracle's fp64 matmul of the de-quantized
operands: relative Frobenius error <= 1e-3 (the tolerance the target states); bit-exact in the
special cases where every partial sum is exactly representable."""
import numpy as np
import pytest
import torch

from tests.util import make_input, to_oracle

pytestmark = pytest.mark.gpu
REL_FRO_TOL = 1e-3


@pytest.fixture(scope="module")
def K():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from quartet_amd import kernels
    return kernels


def _quant(oracle, rows, cols, mode, seed, scale=1.0):
    x = make_input(rows, cols, torch.bfloat16, seed=seed, scale=scale)
    q = oracle.quantize(to_oracle(x), 32, mode=mode)
    return q["codes"], q["scales"]


@pytest.mark.parametrize("M,N,K_", [(128, 128, 128), (256, 384, 512), (96, 160, 224), (32, 32, 32), (1000, 72, 1728)])
def test_gemm_against_fp64_matmul(oracle, K, M, N, K_):
    print(f"case gemm {M}x{N}x{K_}", flush=True)
    dev = torch.device("cuda:0")
    ac, as_ = _quant(oracle, M, K_, oracle.QUEST_RTN, 1)
    bc, bs = _quant(oracle, N, K_, oracle.ABSMAX_RTN, 2, scale=0.02)
    d = float(oracle.FOUR_THIRDS)
    want = oracle.gemm_tn(ac, as_, bc, bs, alpha=1.0, b_post=d)
    args = [torch.from_numpy(t).to(dev) for t in (ac, as_, bc, bs)]
    got32 = K.gemm_mxfp4_tn(*args, alpha=d, out_dtype=torch.float32)
    got16 = K.gemm_mxfp4_tn(*args, alpha=d, out_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    g = got32.cpu().numpy().astype(np.float64)
    rel = np.linalg.norm(g - want) / np.linalg.norm(want)
    assert rel <= REL_FRO_TOL, rel
    assert rel <= 1e-5, rel  # fp32 accumulation of exact products: far inside the stated tolerance
    # the bf16 output is the same accumulator rounded once
    assert torch.equal(got16.cpu(), got32.cpu().to(torch.bfloat16))


def test_gemm_bit_exact_when_sums_are_exact(oracle, K):
    # all scales equal: products are multiples of 1/4 below 2^24 -> every fp32 partial sum is exact
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(0)
    M, N, K_ = 160, 96, 640
    ac = rng.integers(0, 256, (M, K_ // 2), dtype=np.uint8)
    bc = rng.integers(0, 256, (N, K_ // 2), dtype=np.uint8)
    as_ = np.full((M, K_ // 32), 127, dtype=np.uint8)
    bs = np.full((N, K_ // 32), 126, dtype=np.uint8)
    want = oracle.gemm_tn(ac, as_, bc, bs)
    got = K.gemm_mxfp4_tn(*[torch.from_numpy(t).to(dev) for t in (ac, as_, bc, bs)], alpha=1.0, out_dtype=torch.float32)
    assert np.array_equal(got.cpu().numpy().astype(np.float64), want)


def test_gemm_one_hot_operand_selects_single_products(oracle, K):
    dev = torch.device("cuda:0")
    M, N, K_ = 64, 64, 256
    bc, bs = _quant(oracle, N, K_, oracle.QUEST_RTN, 7)
    ac = np.zeros((M, K_ // 2), dtype=np.uint8)
    as_ = np.full((M, K_ // 32), 127, dtype=np.uint8)
    ks = [(3 * m + 5) % K_ for m in range(M)]
    for m, k in enumerate(ks):
        ac[m, k // 2] = 0x2 << (4 * (k & 1))  # +1.0 at column k
    got = K.gemm_mxfp4_tn(*[torch.from_numpy(t).to(dev) for t in (ac, as_, bc, bs)], alpha=1.0, out_dtype=torch.float32)
    B = oracle.dequantize(bc, bs)
    want = np.stack([B[:, k] for k in ks], axis=0)
    assert np.array_equal(got.cpu().numpy(), want)


def _torch_dequant(codes, scales):
    """E2M1/E8M0 unpacking in plain torch ops (float64), checked against the oracle in the test below."""
    lut = torch.tensor([0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6], dtype=torch.float64, device=codes.device)
    lo, hi = (codes & 15).long(), (codes >> 4).long()
    v = torch.stack([lut[lo], lut[hi]], dim=-1).reshape(codes.shape[0], -1)
    s = torch.exp2(scales.to(torch.float64) - 127.0).repeat_interleave(32, dim=1)
    return v * s


# Shapes the tile kernels serve: a single tile, fewer tiles than CUs, more tiles than CUs (each workgroup walks several
# tiles, with an odd and an even number of scale blocks per tile), K that is a multiple of 128 but not of 512 (padding steps
# on the persistent 256x256 kernel), and K up to 768 (one to six K steps on the 256x128 kernel that runs two workgroups per
# CU, scale dwords per K step).
@pytest.mark.parametrize("M,N,K_", [(256, 256, 512), (512, 768, 1024), (4352, 4352, 512), (4608, 4352, 1024),
                                    (768, 512, 1536), (512, 256, 640), (4352, 4608, 384), (8192, 4096, 2048),
                                    # tiles hanging over the edge of M and/or N (extents multiples of 64, not of 256)
                                    (320, 256, 512), (256, 448, 640), (640, 1920, 640), (1728, 640, 1024), (4416, 4160, 512),
                                    (320, 320, 128), (512, 384, 256), (4352, 4480, 768), (256, 128 + 64, 640),
                                    # K a multiple of 128 that the persistent kernel pads to whole blocks of four steps with
                                    # zero-scale steps: three, two and one real steps in the last block; one tile and many
                                    (512, 768, 1920), (4352, 4608, 3840), (320, 256, 3712), (768, 512, 2944), (4608, 4352, 1920),
                                    # few output tiles, long K: cut into K ranges (split-K) when scratch is offered
                                    (512, 256, 8192), (320, 640, 16384), (1920, 640, 4096),
                                    # K % 128 == 64 (row-major operands): a final half step on the 256x128 kernel; one tile,
                                    # tiles over the edge, one and a half K steps, the 30 M Llama's hidden width
                                    (256, 256, 192), (512, 384, 1728), (320, 448, 320), (4352, 640, 1728), (1216, 4160, 704)])
@pytest.mark.parametrize("exact", [True, False])
def test_gemm_tile_kernels(oracle, K, M, N, K_, exact):
    print(f"case gemm tiles {M}x{N}x{K_} exact={exact}", flush=True)
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(M * 7 + N * 3 + K_)
    ac = torch.randint(0, 256, (M, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    bc = torch.randint(0, 256, (N, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    if exact:  # equal scales: every product is a multiple of 1/4 and every partial sum is exact in fp32
        as_ = torch.full((M, K_ // 32), 127, dtype=torch.uint8, device=dev)
        bs = torch.full((N, K_ // 32), 125, dtype=torch.uint8, device=dev)
    else:
        as_ = torch.randint(118, 132, (M, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
        bs = torch.randint(120, 136, (N, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    A, B = _torch_dequant(ac, as_), _torch_dequant(bc, bs)
    # the unpacking helper itself, on a corner of the operands
    assert np.array_equal(A[:64].cpu().numpy(), oracle.dequantize(ac[:64].cpu().numpy(), as_[:64].cpu().numpy()).astype(np.float64))
    want = A @ B.T
    got32 = K.gemm_mxfp4_tn(ac, as_, bc, bs, alpha=1.0, out_dtype=torch.float32)
    got16 = K.gemm_mxfp4_tn(ac, as_, bc, bs, alpha=1.0, out_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    if exact:
        assert torch.equal(got32.double(), want)
    else:
        rel = float((got32.double() - want).norm() / want.norm())
        assert rel <= 1e-5, rel
    assert torch.equal(got16, got32.to(torch.bfloat16))


@pytest.mark.parametrize("M,N,K_", [(256, 256, 512), (768, 512, 1536), (512, 256, 640), (4352, 4608, 1024), (640, 1920, 640),
                                    (1728, 448, 1024), (512, 768, 1920), (640, 384, 3712), (4352, 512, 3840)])
@pytest.mark.parametrize("a_tiled,b_tiled", [(True, True), (True, False), (False, True)])
def test_gemm_tiled_operands_match_rowmajor(K, M, N, K_, a_tiled, b_tiled):
    print(f"case gemm tiled {M}x{N}x{K_} a={a_tiled} b={b_tiled}", flush=True)
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(M + N + K_)
    ac = torch.randint(0, 256, (M, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    bc = torch.randint(0, 256, (N, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    as_ = torch.randint(118, 132, (M, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    bs = torch.randint(120, 136, (N, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    want = K.gemm_mxfp4_tn(ac, as_, bc, bs, alpha=1.0, out_dtype=torch.float32)
    got = K.gemm_mxfp4_tn(K.tile_codes(ac) if a_tiled else ac, as_, K.tile_codes(bc) if b_tiled else bc, bs, alpha=1.0,
                          out_dtype=torch.float32, a_tiled=a_tiled, b_tiled=b_tiled)
    got16 = K.gemm_mxfp4_tn(K.tile_codes(ac) if a_tiled else ac, as_, K.tile_codes(bc) if b_tiled else bc, bs, alpha=1.0,
                            out_dtype=torch.bfloat16, a_tiled=a_tiled, b_tiled=b_tiled)
    torch.cuda.synchronize()
    # same kernel, same summation order: the layout only changes where the operand bytes are fetched from
    assert torch.equal(got, want)
    assert torch.equal(got16, want.to(torch.bfloat16))


@pytest.mark.parametrize("tiled", [False, True])
def test_gemm_scale_arrays_off_16_byte_alignment(K, tiled):
    """K % 512 == 0 with scale arrays that are 4-byte but not 16-byte aligned: the persistent kernel's 16-byte scale
    requests cannot serve them, the 256x128 kernel (4-byte scale requests, any K % 128 == 0) takes over -- same result,
    row-major or tiled codes."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(77)
    M, N, K_ = 512, 384, 1024
    ac = torch.randint(0, 256, (M, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    bc = torch.randint(0, 256, (N, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    as_ = torch.randint(118, 132, (M, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    bs = torch.randint(120, 136, (N, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    want = K.gemm_mxfp4_tn(ac, as_, bc, bs, alpha=1.0, out_dtype=torch.float32)

    def shifted(t):
        buf = torch.empty(t.numel() + 4, dtype=torch.uint8, device=dev)
        view = buf[4:].view(t.shape)
        view.copy_(t)
        assert view.data_ptr() % 16 == 4
        return view
    a_in, b_in = (K.tile_codes(ac), K.tile_codes(bc)) if tiled else (ac, bc)
    got = K.gemm_mxfp4_tn(a_in, shifted(as_), b_in, shifted(bs), alpha=1.0, out_dtype=torch.float32, a_tiled=tiled, b_tiled=tiled)
    # another kernel, another order of the partial sums: equal to fp32 rounding, not bit for bit
    rel = float((got.double() - want.double()).norm() / want.double().norm())
    assert rel <= 1e-6, rel


# the product with the masked inverse rotation in its epilogue: one tile, several tiles per workgroup, tiles over the edge of
# M and N, K with padding steps, both operand layouts
@pytest.mark.parametrize("M,N,K_", [(256, 256, 1024), (512, 768, 1536), (4352, 4608, 1024), (320, 448, 1920), (8192, 4096, 2048)])
@pytest.mark.parametrize("tiled", [False, True])
def test_product_with_the_inverse_rotation_in_its_epilogue(oracle, K, M, N, K_, tiled):
    """qm_gemm_mxfp4_tn_rotated against the two calls it replaces (bf16 product, then masked_hadamard_bwd): the same
    bf16-rounded, masked tile is rotated, only the fp32 arithmetic inside a group's sum differs (the matrix instruction's
    order; with a bf16 scale dtype the factor 32^-1/2 multiplies the terms, as in the reference's bf16 product, instead of
    the sum), so all but a few elements in a million are identical; and against the float64 evaluation of the definition."""
    print(f"case rotated product {M}x{N}x{K_} tiled={tiled}", flush=True)
    if tiled and (M % 128 or N % 128):
        pytest.skip("the tiled layout needs rows in blocks of 128")
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(M + 3 * N + K_)
    ac = torch.randint(0, 256, (M, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    bc = torch.randint(0, 256, (N, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    as_ = torch.randint(118, 132, (M, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    bs = torch.randint(120, 136, (N, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    keep = torch.randint(0, 256, (M, N // 8), generator=g, dtype=torch.uint8)
    keep |= torch.randint(0, 256, (M, N // 8), generator=g, dtype=torch.uint8)      # three quarters of the bits set
    keep = keep.to(dev)
    signs = int(torch.randint(0, 2 ** 31, (1,), generator=g)) * 2 + 1
    alpha = 16.0 / 9.0
    assert K.gemm_fuses_rotation(as_, bs, M, N, K_)
    at, bt = (K.tile_codes(ac), K.tile_codes(bc)) if tiled else (ac, bc)
    for sd in (torch.bfloat16, torch.float32):
        got = K.gemm_mxfp4_tn_rotated(at, as_, bt, bs, keep, alpha, sd, signs, a_tiled=tiled, b_tiled=tiled)
        plain = K.gemm_mxfp4_tn(at, as_, bt, bs, alpha, torch.bfloat16, a_tiled=tiled, b_tiled=tiled)
        two = K.masked_hadamard_bwd(plain, 32, sd, signs, keep)
        torch.cuda.synchronize()
        differ = got != two
        frac = float(differ.float().mean())
        print(f"  scale dtype {sd}: {int(differ.sum())} of {differ.numel()} elements differ from the two-call result", flush=True)
        assert frac < 1e-4
        # where they differ: by a bf16 rounding step at the element's size, or -- where a group's terms cancel -- by the fp32
        # rounding of its partial sums, which is tiny against the terms themselves
        step = two.float().abs() * 2.0 ** -7 + float(plain.float().abs().max()) * 2.0 ** -18
        assert bool(((got.float() - two.float()).abs() <= step)[differ].all())
        # the definition in float64 on sampled rows: bf16(alpha A B^T) * keep, groups of 32 times the signed Sylvester matrix
        rows = torch.cat([torch.tensor([0, M - 1]), torch.randint(0, M, (14,), generator=g)]).to(dev)
        A = _torch_dequant(ac[rows], as_[rows])
        B = _torch_dequant(bc, bs)
        y = (alpha * (A @ B.T)).to(torch.float32).to(torch.bfloat16).double()
        bits = ((keep[rows].long()[:, :, None] >> torch.arange(8, device=dev)) & 1).reshape(len(rows), N).double()
        n = torch.arange(32, device=dev)
        syl = 1.0 - 2.0 * (torch.tensor([[bin(int(a & b)).count("1") & 1 for b in range(32)] for a in range(32)], device=dev)).double()
        sgn = 1.0 - 2.0 * ((signs >> n) & 1).double()
        c = float(torch.tensor(32 ** -0.5).to(sd))
        want = (((y * bits).view(len(rows), N // 32, 32) * sgn) @ syl.T).reshape(len(rows), N) * c
        rel = float((got[rows].double() - want).norm() / want.norm())
        assert rel < 4e-3, rel     # the bf16 rounding of the result: 2^-9 relative per element


def test_split_k_is_offered_and_reproducible(K):
    from quartet_amd import _lib
    L = _lib.lib()
    assert L.qm_gemm_workspace_bytes(512, 256, 8192) > 0          # 2 tiles, 64 K steps
    assert L.qm_gemm_workspace_bytes(8192, 4096, 4096) == 0       # 512 tiles fill the chip
    assert L.qm_gemm_workspace_bytes(512, 256, 640) == 0          # K not a multiple of 512
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(5)
    M, N, K_ = 512, 256, 8192
    ac = torch.randint(0, 256, (M, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    bc = torch.randint(0, 256, (N, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    as_ = torch.randint(118, 132, (M, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    bs = torch.randint(120, 136, (N, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    a = K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.5, torch.float32)
    b = K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.5, torch.float32)
    plain = K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.5, torch.float32, split_k=False)
    torch.cuda.synchronize()
    assert torch.equal(a, b)  # fixed reduction order
    rel = float((a.double() - plain.double()).norm() / plain.double().norm())
    assert rel < 1e-6, rel


def test_matrix_instruction_loop_reports_its_instruction_count(K):
    """The matrix-instruction loop (a measurement aid) reports how many instructions it issued, and leaves the product's
    results alone."""
    dev = torch.device("cuda:0")
    g = torch.Generator(device="cpu").manual_seed(5)
    M, N, K_ = 512, 768, 1024
    ac = torch.randint(0, 256, (M, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    bc = torch.randint(0, 256, (N, K_ // 2), generator=g, dtype=torch.uint8).to(dev)
    as_ = torch.randint(120, 130, (M, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    bs = torch.randint(120, 130, (N, K_ // 32), generator=g, dtype=torch.uint8).to(dev)
    plain = K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.0, torch.bfloat16)
    buf = torch.randint(0, 256, (16 << 20,), generator=g, dtype=torch.uint8).to(dev)
    n = K.mfma_only(buf, 10)
    torch.cuda.synchronize()
    assert n > 0 and n % (4 * 10 * 16) == 0
    after = K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.0, torch.bfloat16)
    assert torch.equal(after, plain)


def test_tile_phase_stamps_of_the_persistent_kernel():
    """The measurement instantiation of the persistent tile kernel (qm_diag_gemm_tile_phases) computes the same product,
    bit for bit, and its per-workgroup stamps are ordered: entry <= loop start < K loop end < epilogue end < ... for as
    many tiles as the workgroup walked; together the workgroups walked every tile once."""
    from quartet_amd import kernels as K, _lib
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(17)
    M, N, Kd = 2048, 2816, 1024    # 8 x 11 tiles: fewer tiles than CUs, then one per workgroup
    for M, N in ((2048, 2816), (8192, 4096)):
        ac = torch.randint(0, 256, (M, Kd // 2), generator=g, dtype=torch.uint8).to(dev)
        as_ = torch.randint(118, 130, (M, Kd // 32), generator=g, dtype=torch.uint8).to(dev)
        bc = torch.randint(0, 256, (N, Kd // 2), generator=g, dtype=torch.uint8).to(dev)
        bs = torch.randint(118, 130, (N, Kd // 32), generator=g, dtype=torch.uint8).to(dev)
        want = K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.5, torch.bfloat16, split_k=False)
        got, stamps = K.gemm_tile_phases(ac, as_, bc, bs, 1.5)
        assert torch.equal(got, want)
        # the instantiation with the masked inverse rotation in its epilogue: the fused product, bit for bit
        keep = torch.randint(0, 256, (M, N // 8), generator=g, dtype=torch.uint8).to(dev)
        got_rot, stamps_rot = K.gemm_tile_phases(ac, as_, bc, bs, 1.5, maskbits=keep)
        assert torch.equal(got_rot, K.gemm_mxfp4_tn_rotated(ac, as_, bc, bs, keep, 1.5, torch.bfloat16, None))
        assert stamps_rot.shape == stamps.shape
        tiles = 0
        for row in stamps.tolist():
            assert 0 < row[0] <= row[1]
            prev = row[1]
            for i in range(2, K.PHASE_STAMPS - 1, 2):
                if row[i] == 0:
                    assert row[i + 1] == 0
                    break
                assert prev < row[i] < row[i + 1]
                prev = row[i + 1]
                tiles += 1
        assert tiles == (M // 256) * (N // 256)
    with pytest.raises(_lib.QuartetHipError):   # K % 512 != 0: not served
        K.gemm_tile_phases(ac[:, :320].contiguous(), as_[:, :20].contiguous(), bc[:, :320].contiguous(), bs[:, :20].contiguous())


# ---- MXFP4 x bf16 "NN" product (the scheme that quantizes only the error signal) -----------------------------------
def _nn_reference(oracle, ac, as_, b, alpha):
    """float64 product of the de-quantized codes with the bf16 operand: the reference's `Q(e) @ w` without any rounding."""
    a = oracle.dequantize(ac, as_).astype(np.float64)
    return alpha * (a @ b.float().numpy().astype(np.float64))


@pytest.mark.parametrize("M,N,K_", [(128, 128, 64), (256, 384, 512), (96, 200, 192), (1000, 72, 1728), (640, 1728, 2048)])
def test_fp4_bf16_product_against_fp64_matmul(oracle, K, M, N, K_):
    """A packed (absmax codes of a small-valued tensor, like an error signal), B bf16 [K, N] as it lies in memory."""
    print(f"case fp4 x bf16 product {M}x{N}x{K_}", flush=True)
    dev = torch.device("cuda:0")
    ac, as_ = _quant(oracle, M, K_, oracle.ABSMAX_RTN, 11, scale=1e-3)
    b = make_input(K_, N, torch.bfloat16, seed=12, scale=0.02)
    d = float(oracle.FOUR_THIRDS)
    want = _nn_reference(oracle, ac, as_, b, d)
    act, ast, bt = torch.from_numpy(ac).to(dev), torch.from_numpy(as_).to(dev), b.to(dev)
    got32 = K.gemm_mxfp4_bf16_nn(act, ast, bt, alpha=d, out_dtype=torch.float32)
    got16 = K.gemm_mxfp4_bf16_nn(act, ast, bt, alpha=d, out_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    rel = np.linalg.norm(got32.cpu().numpy().astype(np.float64) - want) / np.linalg.norm(want)
    assert rel <= 1e-5, rel          # exact decode, exact bf16 products, fp32 accumulation
    assert torch.equal(got16.cpu(), got32.cpu().to(torch.bfloat16))


@pytest.mark.parametrize("M,N,K_", [(192, 136, 448), (320, 264, 448), (512, 512, 64), (260, 256, 320)])
def test_fp4_bf16_product_bit_exact_when_sums_are_exact(oracle, K, M, N, K_):
    """Random code bytes with one common scale against small integers: every partial sum is a multiple of 1/2 below 2^24,
    so the fp32 result must equal the float64 product whatever order the contraction index is walked in.  Shapes of the
    128 x 128 kernel and of the 256 x 256 kernel (with tiles hanging over both edges, one to five K steps)."""
    print(f"case fp4 x bf16 exact sums {M}x{N}x{K_}", flush=True)
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(3)
    ac = rng.integers(0, 256, (M, K_ // 2), dtype=np.uint8)
    as_ = np.full((M, K_ // 32), 127, dtype=np.uint8)
    b = torch.from_numpy(rng.integers(-8, 9, (K_, N)).astype(np.float32)).to(torch.bfloat16)
    want = _nn_reference(oracle, ac, as_, b, 1.0)
    got = K.gemm_mxfp4_bf16_nn(torch.from_numpy(ac).to(dev), torch.from_numpy(as_).to(dev), b.to(dev), 1.0, torch.float32)
    assert np.array_equal(got.cpu().numpy().astype(np.float64), want)


@pytest.mark.parametrize("M,N,K_", [(256, 128, 128), (512, 264, 256)])
def test_fp4_bf16_product_selects_rows_and_columns(oracle, K, M, N, K_):
    """One +1.0 per row of A at a known k (every k of a K step occurs, per-group scales differ) returns row k of B times
    the group's scale: pins the order in which lanes, matrix instructions and the transposing LDS read walk k (both
    kernels)."""
    print(f"case fp4 x bf16 selection {M}x{N}x{K_}", flush=True)
    dev = torch.device("cuda:0")
    ac = np.zeros((M, K_ // 2), dtype=np.uint8)
    as_ = (120 + (np.arange(M)[:, None] + np.arange(K_ // 32)[None, :]) % 12).astype(np.uint8)
    ks = [(m * 5 + 3) % K_ for m in range(M)]
    assert set(ks) == set(range(K_))
    for m, k in enumerate(ks):
        ac[m, k // 2] = 0x2 << (4 * (k & 1))
    b = make_input(K_, N, torch.bfloat16, seed=5, scale=1.0, outlier_frac=0)
    got = K.gemm_mxfp4_bf16_nn(torch.from_numpy(ac).to(dev), torch.from_numpy(as_).to(dev), b.to(dev), 1.0, torch.float32)
    bf = b.float().numpy()
    want = np.stack([bf[k] * np.float32(2.0) ** (int(as_[m, k // 32]) - 127) for m, k in enumerate(ks)])
    assert np.array_equal(got.cpu().numpy(), want)


def test_fp4_bf16_product_rejects_what_it_does_not_serve(K):
    from quartet_amd import _lib
    dev = torch.device("cuda:0")
    a = torch.zeros(64, 48, dtype=torch.uint8, device=dev)      # K = 96: not a multiple of 64
    s = torch.zeros(64, 3, dtype=torch.uint8, device=dev)
    with pytest.raises(_lib.QuartetHipError, match="multiple of 64"):
        K.gemm_mxfp4_bf16_nn(a, s, torch.zeros(96, 64, dtype=torch.bfloat16, device=dev))
    with pytest.raises(_lib.QuartetHipError, match="bf16"):
        K.gemm_mxfp4_bf16_nn(a, s, torch.zeros(96, 64, dtype=torch.float32, device=dev))
