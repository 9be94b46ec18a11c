"""CPU tests of the C ABI: the shared library loads, exports exactly what include/quartet_hip.h declares, its
host-only entry points work without a GPU, and argument validation answers with error codes and messages
(no kernel is launched here)."""
import ctypes
import os
import re

import pytest

from quartet_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "quartet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"^\s*(?:const\s+char\s*\*|int|int64_t|size_t)\s+(qm_\w+)\s*\(", text, flags=re.M))


def test_library_exports_every_declared_function():
    names = declared_functions()
    assert len(names) >= 13
    assert names == set(_lib.EXPORTS), names ^ set(_lib.EXPORTS)
    L = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert getattr(L, name) is not None


def test_host_only_entry_points():
    L = _lib.lib()
    assert L.qm_version() == 15
    T, I, O = 256, 128, 384
    off = (ctypes.c_size_t * 3)()
    for rows, cols in ((T, I), (O, I)):
        total = L.qm_packed_operand_bytes(rows, cols)
        assert L.qm_packed_operand_offsets(rows, cols, off) == 0
        sizes = [rows * cols // 2, rows * cols // 32, rows * cols // 8]
        # codes, scales, mask bits in this order, each 256-byte aligned, none overlapping, all inside the buffer
        assert off[0] == 0
        for k in range(3):
            assert off[k] % 256 == 0
            assert off[k] + sizes[k] <= (off[k + 1] if k < 2 else total)
    assert L.qm_packed_operand_bytes(T, 100) == 0                       # cols not a multiple of 32
    assert L.qm_packed_operand_offsets(T, 100, off) != 0 and b"qm_packed_operand_offsets" in L.qm_last_error()
    assert L.qm_packed_operand_offsets(T, I, None) != 0
    assert L.qm_linear_backward_workspace_bytes(T, I, O, _lib.QM_BF16) > 0
    assert L.qm_linear_backward_workspace_bytes(T, I, 100, _lib.QM_BF16) == 0
    assert L.qm_linear_backward_workspace_bytes(T, I, O, 7) == 0
    assert L.qm_gemm_workspace_bytes(256, 256, 100) == 0                # K not a multiple of 32


@pytest.mark.parametrize("call,needle", [
    (lambda L: L.qm_quantize_mxfp4(None, 0, 4, 30, 32, None, 0, 0, None, 0, None, None, None, None, 0, None), b"multiple of hadamard_dim"),
    (lambda L: L.qm_quantize_mxfp4(None, 5, 4, 32, 32, None, 0, 0, None, 0, None, None, None, None, 0, None), b"x_dtype"),
    (lambda L: L.qm_quantize_mxfp4(None, 0, 4, 32, 48, None, 0, 0, None, 0, None, None, None, None, 0, None), b"hadamard_dim"),
    (lambda L: L.qm_quantize_mxfp4(None, 0, 4, 32, 32, None, 9, 0, None, 0, None, None, None, None, 0, None), b"mode"),
    (lambda L: L.qm_quantize_mxfp4(None, 0, 4, 32, 32, None, 0, 0, None, 0, None, None, None, None, 3, None), b"codes_layout"),
    (lambda L: L.qm_quantize_mxfp4(None, 0, 4, 32, 32, None, 0, 0, None, 0, None, None, None, None, 0, None), b"non-null"),
    (lambda L: L.qm_requantize_transposed_mxfp4(None, None, 30, 64, 1.0, 0, 32, None, 2, None, 0, None, None, None, 0, 0, None), b"hadamard_dim"),
    (lambda L: L.qm_gemm_mxfp4_tn(None, None, None, None, 64, 64, 48, 1.0, None, 0, 0, 0, None, 0, None), b"qm_gemm_mxfp4_tn"),
    # an output offset by 4 bytes: the tile kernels store 16-byte pieces, so the call is refused before any launch
    (lambda L: L.qm_gemm_mxfp4_tn(0x1000, 0x2000, 0x3000, 0x4000, 256, 256, 128, 1.0, 0x5004, 0, 0, 0, None, 0, None), b"c 16-byte"),
    # a shape of the generic kernel stores single elements: c misaligned for 4 bytes is refused, 4-byte aligned c is not
    (lambda L: L.qm_gemm_mxfp4_tn(0x1000, 0x2000, 0x3000, 0x4000, 96, 256, 128, 1.0, 0x5002, 0, 0, 0, None, 0, None), b"c 16-byte (4-byte"),
    # the FP4 x bf16 product: contraction a multiple of 64, N a multiple of 8, tensors non-null and aligned
    (lambda L: L.qm_gemm_mxfp4_bf16_nn(None, None, None, 64, 64, 96, 1.0, None, 0, None), b"multiple of 64"),
    (lambda L: L.qm_gemm_mxfp4_bf16_nn(None, None, None, 64, 60, 128, 1.0, None, 0, None), b"multiple of 8"),
    (lambda L: L.qm_gemm_mxfp4_bf16_nn(None, None, None, 64, 64, 128, 1.0, None, 0, None), b"null tensor"),
    (lambda L: L.qm_gemm_mxfp4_bf16_nn(0x1000, 0x2000, 0x3008, 64, 64, 128, 1.0, 0x4000, 0, None), b"16-byte"),
    (lambda L: L.qm_gemm_mxfp4_bf16_nn(0x1000, 0x2000, 0x3000, 64, 64, 128, 1.0, 0x4000, 9, None), b"c_dtype"),
    # the product with the inverse rotation in its epilogue: null tensors, shapes the persistent kernel does not serve (a short
    # contraction), misaligned mask bits
    (lambda L: L.qm_gemm_mxfp4_tn_rotated(None, None, None, None, 256, 256, 1024, 1.0, None, 0, 0, None, None, 0, None), b"null tensor"),
    (lambda L: L.qm_gemm_mxfp4_tn_rotated(0x1000, 0x2000, 0x3000, 0x4000, 256, 256, 512, 1.0, 0x5000, 0, 0, 0x6000, None, 0, None), b"not served"),
    (lambda L: L.qm_gemm_mxfp4_tn_rotated(0x1000, 0x2000, 0x3000, 0x4000, 256, 200, 1024, 1.0, 0x5000, 0, 0, 0x6000, None, 0, None), b"not served"),
    (lambda L: L.qm_gemm_mxfp4_tn_rotated(0x1000, 0x2000, 0x3000, 0x4000, 256, 256, 1024, 1.0, 0x5000, 0, 0, 0x6002, None, 0, None), b"4-byte"),
    (lambda L: L.qm_gemm_mxfp4_tn_rotated(0x1000, 0x2000, 0x3000, 0x4000, 256, 256, 1024, 1.0, 0x5000, 0, 0, 0x6000, None, 5, None), b"scale_dtype"),
    (lambda L: L.qm_quantize_mxfp4_dense(None, 0, 4, 40, None, 1, 0, 0, None, None, None, None, 0, None), b"multiple of 32"),
    (lambda L: L.qm_quantize_mxfp4_dense(None, 0, 4, 64, None, 1, 0, 0, None, None, None, None, 0, None), b"non-null"),
    (lambda L: L.qm_quantize_mxfp4_dense(0x1000, 0, 64, 64, 0x2000, 1, 1, 0, 0x3000, 0x4000, None, None, 0, None), b"transposed input needs"),
    (lambda L: L.qm_requantize_transposed_mxfp4_dense(None, None, 64, 64, 1.0, 0, None, 2, 0, None, None, None, 0, 0, None), b"R % 128"),
    (lambda L: L.qm_requantize_transposed_mxfp4_dense(None, None, 128, 64, 1.0, 0, None, 2, 0, None, None, None, 0, 0, None), b"null tensor"),
    (lambda L: L.qm_masked_hadamard_bwd(None, 0, 4, 40, 32, 0, None, None, None, 0, None), b"multiple of hadamard_dim"),
    (lambda L: L.qm_dequantize_mxfp4(None, None, 4, 40, 1.0, None, 0, None), b"C % 32"),
    (lambda L: L.qm_linear_forward(None, 0, None, 0, 64, 40, 64, 32, None, 32, None, None, 0, None, 0, 0, None, 0, 0, None), b"multiple of 32"),
    (lambda L: L.qm_linear_forward(None, 0, None, 0, 64, 64, 64, 32, None, 32, None, None, 0, None, 0, 0, None, 0, 0, None), b"packed operand buffers"),
    (lambda L: L.qm_rmsnorm_quantize_mxfp4(None, 0, None, 0, None, None, 1e-5, 16, 40, None, None, 0, None, 0, None), b"multiple of 32"),
    (lambda L: L.qm_rmsnorm_quantize_mxfp4(None, 0, None, 0, None, None, 1e-5, 20, 128, None, None, 0, None, 1, None), b"tiled codes"),
    (lambda L: L.qm_rmsnorm_quantize_mxfp4(None, 0, None, 0, None, None, 1e-5, 16, 128, None, None, 0, None, 0, None), b"non-null"),
    (lambda L: L.qm_swiglu_quantize_mxfp4(None, 7, 16, 128, None, None, 0, 0, None), b"dtype"),
    (lambda L: L.qm_swiglu_quantize_mxfp4(None, 0, 16, 100, None, None, 0, 0, None), b"multiple of 32"),
    (lambda L: L.qm_swiglu_quantize_mxfp4(None, 0, 16, 128, None, None, 0, 0, None), b"non-null"),
    (lambda L: L.qm_rmsnorm_backward(None, 0, None, 0, None, None, 16, 16384, None, None, 0, None, None, None, None, None, 0, None), b"[32, 8192]"),
    (lambda L: L.qm_rmsnorm_backward(None, 0, None, 0, None, None, 16, 128, None, None, 0, None, None, None, None, None, 0, None), b"dgain"),
    # no rows: pointers are not dereferenced, the misaligned mask-bit pointer is still refused
    (lambda L: L.qm_rmsnorm_backward(None, 0, None, 0, None, None, 0, 128, 0x1001, None, 0, None, None, None, 0x1000, None, 0, None), b"4-byte"),
    (lambda L: L.qm_swiglu_backward(None, 0, None, 0, 16, 30, None, None, 0, None, None), b"multiple of 4"),
    (lambda L: L.qm_swiglu_backward(None, 0, None, 0, 16, 32, None, None, 0, None, None), b"non-null"),
])
def test_rejected_arguments_report_an_error(call, needle):
    L = _lib.lib()
    rc = call(L)
    assert rc < 0
    assert needle in L.qm_last_error(), L.qm_last_error()


def test_empty_shapes_are_accepted_without_touching_pointers():
    L = _lib.lib()
    assert L.qm_quantize_mxfp4(None, 0, 0, 64, 32, None, 0, 0, None, 0, None, None, None, None, 0, None) == 0
    assert L.qm_gemm_mxfp4_tn(None, None, None, None, 0, 64, 64, 1.0, None, 0, 0, 0, None, 0, None) == 0
    assert L.qm_gemm_mxfp4_bf16_nn(None, None, None, 0, 64, 64, 1.0, None, 0, None) == 0
    assert L.qm_gemm_mxfp4_tn_rotated(None, None, None, None, 0, 256, 1024, 1.0, None, 0, 0, None, None, 0, None) == 0
    assert L.qm_linear_forward(None, 0, None, 0, 0, 64, 64, 32, None, 32, None, None, 0, None, 0, 0, None, 0, 0, None) == 0
    assert L.qm_rmsnorm_quantize_mxfp4(None, 0, None, 0, None, None, 1e-5, 0, 64, None, None, 0, None, 0, None) == 0
    assert L.qm_swiglu_quantize_mxfp4(None, 0, 0, 64, None, None, 0, 0, None) == 0
    assert L.qm_swiglu_backward(None, 0, None, 0, 0, 64, None, None, 0, None, None) == 0


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libquartet_hip.so"))
    with pytest.raises(_lib.QuartetHipError, match="no CPU fallback"):
        _lib.lib()
