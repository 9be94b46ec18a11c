"""CPU tests of the ``quartet::`` operator registrations: names, shape functions, the sign reader for dense
rotation matrices, and the refusal to run without a GPU."""
import pytest
import torch

import quartet_amd.ops as ops
from quartet_amd.quantizers.mxfp4 import sylvester_matrix

OPERATORS = ["fusedQuantizeMx_op", "fusedQuantizeMxAbsMax_op", "backward_t_bf16_op", "backward_qt_bf16_op",
             "matmul_mxf4_bf16_tn_op", "maskedHadamardBwd_op"]


def meta(shape, dtype):
    return torch.empty(shape, dtype=dtype, device="meta")


@pytest.mark.parametrize("name", OPERATORS)
def test_operator_is_registered_in_quartet_namespace(name):
    assert hasattr(torch.ops.quartet, name)


def test_shape_functions_follow_the_packed_format():
    M, Kd = 96, 256
    x, h = meta((M, Kd), torch.bfloat16), meta((32, 32), torch.bfloat16)
    c, s, m = torch.ops.quartet.fusedQuantizeMx_op(x, h, True)
    assert (c.shape, s.shape, m.shape) == ((M, Kd // 2), (M, Kd // 32), (M, Kd // 8))
    assert c.dtype == s.dtype == m.dtype == torch.uint8
    assert torch.ops.quartet.fusedQuantizeMx_op(x, h, False)[2].numel() == 0
    c, s = torch.ops.quartet.fusedQuantizeMxAbsMax_op(x, h, True)
    assert (c.shape, s.shape) == ((M, Kd // 2), (M, Kd // 32))
    ct, st = torch.ops.quartet.backward_t_bf16_op(x, h)
    assert (ct.shape, st.shape) == ((Kd, M // 2), (Kd, M // 32))
    cq, sq = torch.ops.quartet.backward_qt_bf16_op(c, s, h, meta((1,), torch.float32))
    assert (cq.shape, sq.shape) == ((Kd, M // 2), (Kd, M // 32))
    y = torch.ops.quartet.matmul_mxf4_bf16_tn_op(c, meta((40, Kd // 2), torch.uint8), s, meta((40, Kd // 32), torch.uint8),
                                                 meta((1,), torch.float32))
    assert y.shape == (M, 40) and y.dtype == torch.bfloat16
    g = torch.ops.quartet.maskedHadamardBwd_op(x, m, h)
    assert g.shape == x.shape and g.dtype == x.dtype


def test_whole_linear_traces_on_fake_tensors():
    from torch._subclasses.fake_tensor import FakeTensorMode
    with FakeTensorMode():
        x = torch.empty(4, 64, 128, device="cuda", dtype=torch.bfloat16)
        w = torch.empty(96, 128, device="cuda", dtype=torch.bfloat16)
        h = torch.empty(32, 32, device="cuda", dtype=torch.bfloat16)
        assert ops.PackedLinearFn.apply(x, w, h, h).shape == (4, 64, 96)
        y, packed = ops.packed_forward(x.flatten(end_dim=-2), w, h)
        gx, gw = ops.packed_backward(torch.empty_like(y), packed, h, h)
        assert gx.shape == (256, 128) and gw.shape == w.shape and gx.dtype == gw.dtype == torch.bfloat16


@pytest.mark.parametrize("hd", [32, 64, 128])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sign_reader_recovers_negated_columns(hd, dtype):
    g = torch.Generator().manual_seed(hd)
    signs = torch.randint(0, 2, (hd,), generator=g) * 2.0 - 1.0
    h = (sylvester_matrix(hd) * torch.tensor(hd ** -0.5) * signs[None, :]).to(dtype)
    want = sum(1 << j for j in range(hd) if signs[j] < 0)
    assert ops.rotation_sign_bits(h) == want
    assert ops.rotation_sign_bits((sylvester_matrix(hd) * torch.tensor(hd ** -0.5)).to(dtype)) == 0


def test_sign_reader_agrees_with_the_quantizer_modules():
    from quartet_amd import AlbertTsengQuantizer
    torch.manual_seed(5)
    q = AlbertTsengQuantizer(hadamard_dim=32, rerotate="signs")
    for _ in range(3):
        q.re_randomize()
        assert ops.rotation_sign_bits(q.hadamard_matrix) == q.sign_bits


def test_sign_reader_rejects_other_matrices():
    h = sylvester_matrix(32) * torch.tensor(32 ** -0.5)
    with pytest.raises(ValueError):
        ops.rotation_sign_bits(torch.linalg.qr(torch.randn(32, 32))[0])
    with pytest.raises(ValueError):
        ops.rotation_sign_bits(h * 2)
    rows_negated = h.clone()
    rows_negated[3] *= -1  # diag(+-1) on the wrong side
    with pytest.raises(ValueError):
        ops.rotation_sign_bits(rows_negated)
    with pytest.raises(ValueError):
        ops.rotation_sign_bits(torch.eye(16))
    with pytest.raises(ValueError):
        ops.rotation_sign_bits(h[:, :16])


def test_sign_reader_sees_in_place_updates():
    h = sylvester_matrix(32) * torch.tensor(32 ** -0.5)
    assert ops.rotation_sign_bits(h) == 0
    h[:, 5] *= -1
    assert ops.rotation_sign_bits(h) == 1 << 5


def test_operators_have_no_cpu_path():
    h = sylvester_matrix(32) * torch.tensor(32 ** -0.5)
    with pytest.raises(NotImplementedError):
        ops.fusedQuantizeMx_op(torch.zeros(32, 32), h, True)
    with pytest.raises(NotImplementedError):
        ops.matmul_mxf4_bf16_tn_op(torch.zeros(32, 16, dtype=torch.uint8), torch.zeros(32, 16, dtype=torch.uint8),
                                   torch.zeros(32, 1, dtype=torch.uint8), torch.zeros(32, 1, dtype=torch.uint8), torch.ones(1))
