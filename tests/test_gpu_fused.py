"""GPU parity of the producers fused into the activation quantizer (RMSNorm -> F1, SwiGLU -> F1) and of their backward
kernels: packed operands bit-exact against the oracle, whole layers bit-exact against the unfused layer fed with the
oracle's producer output, backward passes against float64 autograd of the reference's formulas."""
import ctypes

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from tests.util import from_oracle_bf16, make_input, sign_int, to_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def q():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    import quartet_amd
    return quartet_amd


def unpack(q, buffer, rows, cols, tiled):
    """(codes, scales, mask bits) of a packed operand buffer as row-major numpy arrays."""
    from quartet_amd import packed as P
    t = P.from_operand_buffer(buffer, rows, cols, tiled, q.QuestMXFP4Quantizer()).to_layout("rowmajor")
    return t.codes.cpu().numpy(), t.scales.cpu().numpy(), t.maskbits.cpu().numpy()


def signs_vector(seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, 2, (32,), generator=g) * 2 - 1


def rel(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm())


# rows x cols: tiled (several groups per lane, a ragged last chunk of 4 groups), and row-major shapes with rows that do
# not fill a workgroup and a single group per row
SHAPES = [(256, 640, True), (512, 1536, True), (64, 4096, True), (100, 96, False), (7, 32, False), (48, 1728, False)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols,tiled", SHAPES)
def test_rmsnorm_quantize_against_oracle(oracle, q, rows, cols, tiled, dtype):
    print(f"case rmsnorm_quantize rows={rows} cols={cols} tiled={tiled} dtype={dtype}", flush=True)
    from quartet_amd import kernels as K
    x = make_input(rows, cols, dtype, seed=rows + cols, scale=3.0, zero_rows=1)
    gain = (1.0 + 0.2 * torch.randn(cols, generator=torch.Generator().manual_seed(1))).float()
    signs = signs_vector(cols)
    eps = 1e-5
    normed, factor = oracle.rmsnorm(to_oracle(x), gain.numpy(), eps)
    want = oracle.quantize(normed, 32, signs=signs.numpy(), mode=oracle.QUEST_RTN, want_mask=True)
    packed, got_factor = K.rmsnorm_quantize(x.to(DEV), gain.to(DEV), eps, sign_int(signs), tiled)
    assert np.array_equal(got_factor.cpu().numpy().view(np.uint32), factor.view(np.uint32))
    codes, scales, mask = unpack(q, packed, rows, cols, tiled)
    assert np.array_equal(scales, want["scales"])
    assert np.array_equal(codes, want["codes"])
    assert np.array_equal(mask, want["mask"])
    # the same packed operand as the stand-alone quantizer produces from the oracle's normalised tensor
    direct = K.quantize_mxfp4(torch.from_numpy(normed).to(DEV), 32, sign_int(signs), K.QM_QUEST_RTN, want_mask=True, tiled=False)
    assert np.array_equal(direct[0].cpu().numpy(), codes) and np.array_equal(direct[2].cpu().numpy(), mask)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,hidden,tiled", SHAPES)
def test_swiglu_quantize_against_oracle(oracle, q, rows, hidden, tiled, dtype):
    print(f"case swiglu_quantize rows={rows} hidden={hidden} tiled={tiled} dtype={dtype}", flush=True)
    from quartet_amd import kernels as K
    h12 = make_input(rows, 2 * hidden, dtype, seed=rows * 3 + hidden, scale=2.0, outlier_frac=1e-3, zero_rows=1)
    h12[-1, :8] = torch.tensor([-200.0, 200.0, -95.0, 95.0, -88.0, 88.0, 0.0, -0.0]).to(dtype)   # e^-x overflows / vanishes
    signs = signs_vector(hidden + 1)
    prod = oracle.swiglu(to_oracle(h12))
    want = oracle.quantize(prod, 32, signs=signs.numpy(), mode=oracle.QUEST_RTN, want_mask=True)
    packed = K.swiglu_quantize(h12.to(DEV), sign_int(signs), tiled)
    codes, scales, mask = unpack(q, packed, rows, hidden, tiled)
    assert np.array_equal(scales, want["scales"])
    assert np.array_equal(codes, want["codes"])
    assert np.array_equal(mask, want["mask"])


@pytest.mark.parametrize("gy_dtype,x_dtype", [(torch.bfloat16, torch.float32), (torch.float32, torch.float32),
                                              (torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("rows,cols", [(256, 640), (1000, 1536), (70, 4096), (3, 32)])
def test_rmsnorm_backward_against_float64_autograd(q, rows, cols, gy_dtype, x_dtype):
    print(f"case rmsnorm_backward rows={rows} cols={cols} gy={gy_dtype} x={x_dtype}", flush=True)
    from quartet_amd import kernels as K
    x = make_input(rows, cols, x_dtype, seed=rows, scale=2.0, outlier_frac=0)
    gy = make_input(rows, cols, gy_dtype, seed=rows + 1, scale=1e-2, outlier_frac=0)
    gain = (1.0 + 0.2 * torch.randn(cols, generator=torch.Generator().manual_seed(2))).float()
    eps = 1e-5
    xd = x.double().requires_grad_(True)
    gd = gain.double().requires_grad_(True)
    y = xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + eps) * gd      # llama.py:64-75 in float64
    y.backward(gy.double())
    factor = torch.rsqrt(x.double().pow(2).mean(-1) + eps).float()
    dx, dgain = K.rmsnorm_backward(gy.to(DEV), x.to(DEV), gain.to(DEV), factor.to(DEV))
    assert dx.dtype == x_dtype and dgain.dtype == torch.float32
    assert rel(dx.cpu(), xd.grad) < (4e-3 if x_dtype == torch.bfloat16 else 2e-6)
    assert rel(dgain.cpu(), gd.grad) < 2e-5
    # reproducible: the column sums are added in a fixed order
    dx2, dgain2 = K.rmsnorm_backward(gy.to(DEV), x.to(DEV), gain.to(DEV), factor.to(DEV))
    assert torch.equal(dgain, dgain2) and torch.equal(dx, dx2)


@pytest.mark.parametrize("g_dtype,h_dtype", [(torch.bfloat16, torch.bfloat16), (torch.float32, torch.float32),
                                             (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("rows,hidden", [(256, 1728), (33, 4096), (5, 32)])
def test_swiglu_backward_against_autograd(q, rows, hidden, g_dtype, h_dtype):
    print(f"case swiglu_backward rows={rows} hidden={hidden} g={g_dtype} h={h_dtype}", flush=True)
    from quartet_amd import kernels as K
    h12 = make_input(rows, 2 * hidden, h_dtype, seed=rows, scale=2.0, outlier_frac=1e-3)
    g = make_input(rows, hidden, g_dtype, seed=rows + 7, scale=1e-2, outlier_frac=0)
    hd_ = h12.double().requires_grad_(True)
    up, gate = hd_.split(hidden, dim=-1)
    (F.silu(up) * gate).backward(g.double())
    got = K.swiglu_backward(g.to(DEV), h12.to(DEV))
    assert got.dtype == h_dtype and got.shape == h12.shape
    tol = 6e-3 if h_dtype == torch.bfloat16 else 2e-6
    assert rel(got[:, :hidden].cpu(), hd_.grad[:, :hidden]) < tol
    assert rel(got[:, hidden:].cpu(), hd_.grad[:, hidden:]) < tol
    if h_dtype == torch.bfloat16:
        # element-wise: within two bf16 steps of autograd run op by op in bf16, as the unfused model does
        hb = h12.clone().to(DEV).requires_grad_(True)
        ub, gb = hb.split(hidden, dim=-1)
        (F.silu(ub) * gb).backward(g.to(DEV).to(torch.bfloat16))
        diff = (got.float() - hb.grad.float()).abs()
        assert bool((diff <= 2.0 ** -6 * hb.grad.float().abs() + 1e-30).all())


def production_layer(q, I, O, dtype):
    return q.QuantizedLinear(I, O, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
                             activation_quantizer=q.QuestMXFP4Quantizer(),
                             gradient_quantizer=q.AlbertTsengQuantizer(stochastic=False, rerotate=None),
                             backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(DEV, dtype)


@pytest.mark.parametrize("dense_w", [False, True])
@pytest.mark.parametrize("autocast", [True, False])
@pytest.mark.parametrize("T,I,O", [(256, 640, 1920), (96, 160, 224)])
def test_rmsnorm_linear_matches_the_unfused_layer(oracle, q, T, I, O, autocast, dense_w):
    """The fused layer against the same layer called on the oracle's normalised tensor: identical packed operands, so
    identical outputs and weight gradients; the gradient w.r.t. x against float64 autograd of RMSNorm applied to the
    unfused layer's input gradient."""
    print(f"case rmsnorm_linear T={T} I={I} O={O} autocast={autocast}", flush=True)
    from quartet_amd.fused import rmsnorm_linear
    from quartet_amd.llama import RMSNorm
    torch.manual_seed(0)
    layer = production_layer(q, I, O, torch.float32)
    if dense_w:   # a weight quantizer holding the dense matrix of rerotate="O32" stays with the fused producer
        layer.weight_quantizer.rerotate = "O32"
        layer.weight_quantizer.re_randomize()
    norm = RMSNorm(I, eps=1e-5).to(DEV)
    with torch.no_grad():
        norm.weight.add_(0.1 * torch.randn(I, device=DEV))
    x = make_input(2 * (T // 2), I, torch.float32, seed=4, scale=2.0).view(2, T // 2, I).to(DEV)
    dy = make_input(T, O, torch.bfloat16 if autocast else torch.float32, seed=5, scale=1e-2, outlier_frac=0).view(2, T // 2, O).to(DEV)
    ctx = (lambda: torch.autocast("cuda", dtype=torch.bfloat16)) if autocast else (lambda: torch.autocast("cuda", enabled=False))

    xf = x.clone().requires_grad_(True)
    with ctx():
        y = rmsnorm_linear(norm, layer, xf)
        y.backward(dy)
    got = (y.detach(), xf.grad, layer.weight.grad.clone(), norm.weight.grad.clone())
    layer.weight.grad = None
    norm.weight.grad = None

    normed, _ = oracle.rmsnorm(x.view(T, I).cpu().numpy(), norm.weight.detach().cpu().numpy(), 1e-5)
    n = torch.from_numpy(normed).view(2, T // 2, I).to(DEV).requires_grad_(True)
    with ctx():
        y_ref = layer(n)
        y_ref.backward(dy)
    assert y.dtype == y_ref.dtype and torch.equal(got[0], y_ref.detach())
    assert torch.equal(got[2], layer.weight.grad)
    xd = x.double().requires_grad_(True)
    gd = norm.weight.detach().double().requires_grad_(True)
    (xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-5) * gd).backward(n.grad.double())
    assert got[1].dtype == torch.float32 and rel(got[1], xd.grad) < 1e-5
    assert rel(got[3], gd.grad) < 1e-4


@pytest.mark.parametrize("dense_w", [False, True])
@pytest.mark.parametrize("autocast", [True, False])
@pytest.mark.parametrize("T,I,O", [(256, 1792, 640), (64, 96, 160)])
def test_swiglu_linear_matches_the_unfused_layer(oracle, q, T, I, O, autocast, dense_w):
    print(f"case swiglu_linear T={T} hidden={I} O={O} autocast={autocast}", flush=True)
    from quartet_amd.fused import swiglu_linear
    torch.manual_seed(0)
    layer = production_layer(q, I, O, torch.float32)
    if dense_w:
        layer.weight_quantizer.rerotate = "O32"
        layer.weight_quantizer.re_randomize()
    dtype = torch.bfloat16 if autocast else torch.float32    # w12's output dtype under autocast
    h12 = make_input(T, 2 * I, dtype, seed=6, scale=2.0).to(DEV)
    dy = make_input(T, O, dtype, seed=7, scale=1e-2, outlier_frac=0).to(DEV)
    ctx = (lambda: torch.autocast("cuda", dtype=torch.bfloat16)) if autocast else (lambda: torch.autocast("cuda", enabled=False))

    hf = h12.clone().requires_grad_(True)
    with ctx():
        y = swiglu_linear(layer, hf)
        y.backward(dy)
    got = (y.detach(), hf.grad, layer.weight.grad.clone())
    layer.weight.grad = None

    prod = oracle.swiglu(to_oracle(h12))
    p = (from_oracle_bf16(prod) if autocast else torch.from_numpy(prod)).to(DEV).requires_grad_(True)
    with ctx():
        y_ref = layer(p)
        y_ref.backward(dy)
    assert torch.equal(got[0], y_ref.detach())
    assert torch.equal(got[2], layer.weight.grad)
    hd_ = h12.double().requires_grad_(True)
    up, gate = hd_.split(I, dim=-1)
    (F.silu(up) * gate).backward(p.grad.double())
    assert got[1].dtype == dtype and rel(got[1], hd_.grad) < (6e-3 if autocast else 1e-5)


def test_fallbacks_keep_the_unfused_composition(q):
    """A layer that is not in its production configuration (or a Hadamard block other than 32) takes the op-by-op
    path and gives what layer(norm(x)) / layer(silu(up) * gate) give."""
    from quartet_amd.fused import rmsnorm_linear, swiglu_linear
    from quartet_amd.llama import RMSNorm
    torch.manual_seed(1)
    plain = q.QuantizedLinear(64, 96, bias=False).to(DEV)            # identity quantizers, plain scheme
    wide = q.QuantizedLinear(128, 96, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(hadamard_dim=64),
                             activation_quantizer=q.QuestMXFP4Quantizer(hadamard_dim=64),
                             gradient_quantizer=q.AlbertTsengQuantizer(hadamard_dim=64, stochastic=False),
                             backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(DEV)
    dense_x = q.QuantizedLinear(128, 96, bias=False, weight_quantizer=q.QuestMXFP4Quantizer(),
                                activation_quantizer=q.QuestMXFP4Quantizer(rerotate="O32"),
                                gradient_quantizer=q.AlbertTsengQuantizer(stochastic=False),
                                backward_scheme=q.BACKWARD_SCHEMES["Q(E)Q(Wt)t_Q(Et)Q(Xt)t"]()).to(DEV)
    dense_x.activation_quantizer.re_randomize()     # the producers rotate by the Hadamard matrix only
    for layer, I in ((plain, 64), (wide, 128), (dense_x, 128)):
        norm = RMSNorm(I).to(DEV)
        x = torch.randn(32, I, device=DEV)
        assert torch.equal(rmsnorm_linear(norm, layer, x), layer(norm(x)))
        h12 = torch.randn(32, 2 * I, device=DEV)
        up, gate = h12.split(I, dim=-1)
        assert torch.equal(swiglu_linear(layer, h12), layer(F.silu(up) * gate))


@pytest.mark.parametrize("autocast", [True, False])
@pytest.mark.parametrize("B,T,n_head,hs", [(2, 64, 5, 128), (3, 40, 2, 32), (1, 16, 3, 8)])
def test_rope_qkv_matches_the_op_by_op_rotation(q, B, T, n_head, hs, autocast):
    """Split + rotate + convert in one kernel against the reference's composition (split, fp32 pairwise rotation,
    autocast's bf16 copies): bit-identical forward and backward -- both evaluate the same fp32 products and sums."""
    print(f"case rope_qkv B={B} T={T} heads={n_head} head_dim={hs} autocast={autocast}", flush=True)
    from quartet_amd.fused import rope_qkv
    from quartet_amd.llama import apply_rotary, rotary_table
    C = n_head * hs
    dtype = torch.bfloat16 if autocast else torch.float32
    table = rotary_table(hs, 2 * T)[:T].to(DEV)
    qkv = make_input(B * T, 3 * C, dtype, seed=B + T, scale=1.5, outlier_frac=0).view(B, T, 3 * C).to(DEV)
    grads = [make_input(B * T, C, dtype, seed=10 + i, scale=1e-2, outlier_frac=0).view(B, T, n_head, hs).to(DEV) for i in range(3)]

    a = qkv.clone().requires_grad_(True)
    with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
        fq, fk, fv = rope_qkv(a, table, n_head)
    torch.autograd.backward([fq, fk, fv], grads)

    b = qkv.clone().requires_grad_(True)
    q0, k0, v0 = b.split(C, dim=2)
    rq, rk = apply_rotary(q0.view(B, T, n_head, hs), k0.view(B, T, n_head, hs), table)
    rq, rk, rv = rq.to(dtype), rk.to(dtype), v0.view(B, T, n_head, hs)      # what attention receives
    torch.autograd.backward([rq, rk, rv], grads)

    assert fq.dtype == dtype and fq.shape == (B, T, n_head, hs) and fq.is_contiguous()
    assert torch.equal(fq, rq) and torch.equal(fk, rk) and torch.equal(fv, rv)
    assert a.grad.dtype == dtype and torch.equal(a.grad, b.grad)
    # a rotation: norms of q and k pairs are preserved up to rounding, position 0 is the identity
    assert torch.equal(fq[:, 0], qkv[:, 0, :C].view(B, n_head, hs))


@pytest.mark.parametrize("g_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,cols", [(128, 640), (37, 96), (16, 4096)])
def test_inverse_rotation_inside_the_backward_kernels(q, rows, cols, g_dtype):
    """The quantizer's straight-through backward (mask, inverse rotation) applied on the fly by the producers' backward
    kernels gives the bits of the stand-alone kernel followed by the plain backward kernel."""
    print(f"case fused inverse rotation rows={rows} cols={cols} g={g_dtype}", flush=True)
    from quartet_amd import kernels as K
    g = make_input(rows, cols, g_dtype, seed=rows + cols, scale=1e-2, outlier_frac=0).to(DEV)
    x = make_input(rows, cols, torch.float32, seed=3, scale=2.0).to(DEV)
    h12 = make_input(rows, 2 * cols, torch.bfloat16 if g_dtype == torch.bfloat16 else torch.float32, seed=4, scale=2.0).to(DEV)
    gain = (1.0 + 0.2 * torch.randn(cols, generator=torch.Generator().manual_seed(2))).float().to(DEV)
    factor = torch.rsqrt(x.double().pow(2).mean(-1) + 1e-5).float()
    mask = torch.randint(0, 256, (rows, cols // 8), dtype=torch.uint8, generator=torch.Generator().manual_seed(5)).to(DEV)
    signs = sign_int(signs_vector(11))
    for scale_dtype in (torch.bfloat16, torch.float32):
        back = K.masked_hadamard_bwd(g, 32, scale_dtype, signs, mask)
        assert back.dtype == g_dtype
        want_dx, want_dg = K.rmsnorm_backward(back, x, gain, factor)
        got_dx, got_dg = K.rmsnorm_backward(g, x, gain, factor, mask, signs, scale_dtype)
        assert torch.equal(got_dx, want_dx) and torch.equal(got_dg, want_dg)
        assert torch.equal(K.swiglu_backward(g, h12, mask, signs, scale_dtype), K.swiglu_backward(back, h12))


def test_producers_on_random_shapes(oracle, q):
    """Seeded sweep over ragged shapes (rows not a multiple of the 4 rows of a workgroup, one to 130 groups per row, so
    one, two and three passes of a wave over its row) for both producers, both dtypes and both code layouts."""
    from quartet_amd import kernels as K
    rng = np.random.default_rng(7)
    for case in range(24):
        groups = int(rng.choice([1, 2, 3, 5, 16, 17, 63, 64, 65, 127, 130]))
        cols = 32 * groups
        tiled = bool(groups % 4 == 0 and rng.integers(2))
        rows = int(rng.integers(1, 12)) * 16 if tiled else int(rng.integers(1, 90))
        dtype = torch.bfloat16 if rng.integers(2) else torch.float32
        signs = signs_vector(case)
        print(f"case sweep {case}: rows={rows} cols={cols} tiled={tiled} {dtype}", flush=True)
        x = make_input(rows, cols, dtype, seed=case, scale=float(rng.uniform(0.01, 50.0)))
        gain = (1.0 + 0.3 * torch.randn(cols, generator=torch.Generator().manual_seed(case))).float()
        normed, factor = oracle.rmsnorm(to_oracle(x), gain.numpy(), 1e-6)
        want = oracle.quantize(normed, 32, signs=signs.numpy(), mode=oracle.QUEST_RTN, want_mask=True)
        packed, got_factor = K.rmsnorm_quantize(x.to(DEV), gain.to(DEV), 1e-6, sign_int(signs), tiled)
        codes, scales, mask = unpack(q, packed, rows, cols, tiled)
        assert np.array_equal(got_factor.cpu().numpy().view(np.uint32), factor.view(np.uint32))
        assert np.array_equal(scales, want["scales"]) and np.array_equal(codes, want["codes"]) and np.array_equal(mask, want["mask"])
        h12 = make_input(rows, 2 * cols, dtype, seed=100 + case, scale=float(rng.uniform(0.1, 8.0)))
        want = oracle.quantize(oracle.swiglu(to_oracle(h12)), 32, signs=signs.numpy(), mode=oracle.QUEST_RTN, want_mask=True)
        codes, scales, mask = unpack(q, K.swiglu_quantize(h12.to(DEV), sign_int(signs), tiled), rows, cols, tiled)
        assert np.array_equal(scales, want["scales"]) and np.array_equal(codes, want["codes"]) and np.array_equal(mask, want["mask"])


def test_residual_gradient_added_inside_the_norm_backward(q):
    """x + f(norm(x)) with the residual taken from the fused function's second output: the same bits as the plain
    composition, whose two gradients of x autograd adds in a kernel of its own."""
    print("case fused residual gradient", flush=True)
    from quartet_amd import kernels as K
    from quartet_amd.fused import rmsnorm_linear
    from quartet_amd.llama import RMSNorm
    torch.manual_seed(0)
    T, I, O = 256, 640, 640
    layer = production_layer(q, I, O, torch.float32)
    norm = RMSNorm(I, eps=1e-5).to(DEV)
    x = make_input(T, I, torch.float32, seed=4, scale=2.0).to(DEV)
    dy = make_input(T, O, torch.float32, seed=5, scale=1e-2, outlier_frac=0).to(DEV)
    outs = []
    for pass_input in (False, True):
        layer.weight.grad = None
        norm.weight.grad = None
        xa = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            if pass_input:
                y, xr = rmsnorm_linear(norm, layer, xa, pass_input=True)
            else:
                y, xr = rmsnorm_linear(norm, layer, xa), xa
            z = xr + y
        z.backward(dy)
        outs.append((z.detach(), xa.grad.clone(), layer.weight.grad.clone(), norm.weight.grad.clone()))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    # kernel level: skip is added after the norm's own gradient, in x's dtype
    gy = make_input(T, I, torch.bfloat16, seed=6, scale=1e-2, outlier_frac=0).to(DEV)
    gain = norm.weight.detach()
    factor = torch.rsqrt(x.double().pow(2).mean(-1) + 1e-5).float()
    skip = make_input(T, I, torch.float32, seed=7, scale=1e-2, outlier_frac=0).to(DEV)
    dx0, dg0 = K.rmsnorm_backward(gy, x, gain, factor)
    dx1, dg1 = K.rmsnorm_backward(gy, x, gain, factor, skip=skip)
    assert torch.equal(dx1, dx0 + skip) and torch.equal(dg0, dg1)


@pytest.mark.parametrize("add_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("rows,cols,tiled", [(256, 640, True), (50, 96, False), (32, 4096, True)])
def test_residual_sum_inside_the_norm_quantizer(q, rows, cols, tiled, add_dtype):
    """x + add formed inside the fused kernel: the sum it writes and the packed operand are those of the plain kernel on
    torch's x + add; the bf16 copy of the backward's dx is dx rounded."""
    print(f"case fused residual sum rows={rows} cols={cols} tiled={tiled} add={add_dtype}", flush=True)
    from quartet_amd import kernels as K
    x = make_input(rows, cols, torch.float32, seed=rows, scale=2.0).to(DEV)
    a = make_input(rows, cols, add_dtype, seed=rows + 1, scale=0.5).to(DEV)
    gain = (1.0 + 0.2 * torch.randn(cols, generator=torch.Generator().manual_seed(2))).float().to(DEV)
    want_sum = x + a
    assert want_sum.dtype == torch.float32
    p0, f0 = K.rmsnorm_quantize(want_sum, gain, 1e-5, 0x1234ABCD, tiled)
    p1, f1, got_sum = K.rmsnorm_quantize(x, gain, 1e-5, 0x1234ABCD, tiled, add=a)
    assert torch.equal(got_sum, want_sum) and torch.equal(f0, f1)
    for u, v in zip(unpack(q, p0, rows, cols, tiled), unpack(q, p1, rows, cols, tiled)):   # (the buffers' padding is not set)
        assert np.array_equal(u, v)
    gy = make_input(rows, cols, torch.bfloat16, seed=9, scale=1e-2, outlier_frac=0).to(DEV)
    dx, dg = K.rmsnorm_backward(gy, want_sum, gain, f0)
    dx2, dg2, low = K.rmsnorm_backward(gy, want_sum, gain, f0, want_bf16_copy=True)
    assert torch.equal(dx, dx2) and torch.equal(dg, dg2) and torch.equal(low, dx.to(torch.bfloat16))


def test_block_with_deferred_residual_sums_matches_the_plain_block(q):
    """Two fused blocks chained through `pending` against the same blocks with every residual sum done by torch."""
    print("case fused blocks with pending sums", flush=True)
    from quartet_amd import llama as L
    from quartet_amd.fused import rmsnorm_linear
    torch.manual_seed(0)
    det = dict(g_quant_kwargs={"hadamard_dim": 32, "stochastic": False, "rerotate": None})
    cfg = L.LlamaConfig(vocab_size=128, sequence_length=64, n_layer=2, n_head=2, n_embd=256, multiple_of=128, **det)
    model = L.Llama(cfg).to(DEV)
    idx = torch.randint(0, 128, (4, 64), device=DEV)
    tgt = torch.randint(0, 128, (4, 64), device=DEV)

    def run(plain_sums):
        model.zero_grad(set_to_none=True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            if not plain_sums:
                loss = model(idx, targets=tgt)["loss"]
            else:   # the fused kernels for norm, SwiGLU and rotary, but x + branch as separate torch adds
                x = model.transformer.wte(idx)
                table = model.freqs_cis[:64]
                for blk in model.transformer.h:
                    a, _ = blk.attn(x, table, norm=blk.ln_1)
                    x = x + a
                    m, _ = blk.mlp(x, norm=blk.ln_2)
                    x = x + m
                logits = model.lm_head(model.transformer.ln_f(x))
                loss = F.cross_entropy(logits.view(-1, logits.size(-1)), tgt.view(-1), ignore_index=-1)
            loss.backward()
        return loss.detach().clone(), {n: p.grad.clone() for n, p in model.named_parameters()}

    l0, g0 = run(False)
    l1, g1 = run(True)
    assert torch.equal(l0, l1)
    for n in g0:
        assert torch.equal(g0[n], g1[n]), n
