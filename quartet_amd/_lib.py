"""ctypes binding of libquartet_hip.so (the C ABI declared in include/quartet_hip.h).

There is no fallback: if the shared library is missing the import of this module's ``lib()``
raises, so no caller can silently run without the HIP kernels."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libquartet_hip.so")

QM_BF16, QM_F32 = 0, 1
QM_QUEST_RTN, QM_ABSMAX_RTN, QM_ABSMAX_SR, QM_QUEST_SR = 0, 1, 2, 3
QM_LAYOUT_ROWMAJOR, QM_LAYOUT_TILED = 0, 1

EXPORTS = (
    "qm_version",
    "qm_last_error",
    "qm_quantize_mxfp4",
    "qm_requantize_transposed_mxfp4",
    "qm_quantize_mxfp4_dense",
    "qm_requantize_transposed_mxfp4_dense",
    "qm_gemm_mxfp4_tn",
    "qm_masked_hadamard_bwd",
    "qm_dequantize_mxfp4",
    "qm_gemm_workspace_bytes",
    "qm_diag_mfma_only",
    "qm_diag_gemm_tile_phases",
    "qm_gemm_mxfp4_bf16_nn",
    "qm_gemm_noalloc_scratch_bytes",
    "qm_gemm_mxfp4_tn_noalloc",
    "qm_gemm_noalloc_prepare",
    "qm_gemm_fuses_rotation",
    "qm_gemm_mxfp4_tn_rotated",
    "qm_packed_operand_bytes",
    "qm_packed_operand_offsets",
    "qm_linear_backward_workspace_bytes",
    "qm_linear_forward",
    "qm_linear_backward",
    "qm_linear_backward_seeded",
    "qm_rmsnorm_quantize_mxfp4",
    "qm_swiglu_quantize_mxfp4",
    "qm_rmsnorm_backward_workspace_bytes",
    "qm_rmsnorm_backward",
    "qm_swiglu_backward",
    "qm_rope_split_qkv",
    "qm_rope_merge_qkv_grad",
)

_lib = None


class QuartetHipError(RuntimeError):
    pass


def lib():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise QuartetHipError(
            f"{LIB_PATH} is missing: build it with `make -C quartet_amd/csrc` (or __graft_entry__.build()); "
            "there is no CPU fallback for the quantized-linear path")
    L = ctypes.CDLL(LIB_PATH)
    vp, i32, i64, u64, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_uint64, ctypes.c_float
    L.qm_version.restype = i32
    L.qm_version.argtypes = []
    L.qm_last_error.restype = ctypes.c_char_p
    L.qm_last_error.argtypes = []
    L.qm_quantize_mxfp4.restype = i32
    L.qm_quantize_mxfp4.argtypes = [vp, i32, i64, i64, i32, vp, i32, i32, vp, u64, vp, vp, vp, vp, i32, vp]
    L.qm_requantize_transposed_mxfp4.restype = i32
    L.qm_requantize_transposed_mxfp4.argtypes = [vp, vp, i64, i64, f32, i32, i32, vp, i32, vp, u64, vp, vp, vp, i32, i32, vp]
    L.qm_quantize_mxfp4_dense.restype = i32
    L.qm_quantize_mxfp4_dense.argtypes = [vp, i32, i64, i64, vp, i32, i32, u64, vp, vp, vp, vp, i32, vp]
    L.qm_requantize_transposed_mxfp4_dense.restype = i32
    L.qm_requantize_transposed_mxfp4_dense.argtypes = [vp, vp, i64, i64, f32, i32, vp, i32, u64, vp, vp, vp, i32, i32, vp]
    L.qm_gemm_mxfp4_tn.restype = i32
    L.qm_gemm_mxfp4_tn.argtypes = [vp, vp, vp, vp, i64, i64, i64, f32, vp, i32, i32, i32, vp, ctypes.c_size_t, vp]
    L.qm_diag_gemm_tile_phases.restype = i32
    L.qm_diag_gemm_tile_phases.argtypes = [vp, vp, vp, vp, i64, i64, i64, f32, vp, i32, i32, vp, vp, ctypes.c_size_t, vp]
    L.qm_diag_mfma_only.restype = i64
    L.qm_diag_mfma_only.argtypes = [vp, ctypes.c_size_t, vp, ctypes.c_size_t, i32, vp]
    L.qm_gemm_workspace_bytes.restype = ctypes.c_size_t
    L.qm_gemm_workspace_bytes.argtypes = [i64, i64, i64]
    L.qm_gemm_noalloc_scratch_bytes.restype = ctypes.c_size_t
    L.qm_gemm_noalloc_scratch_bytes.argtypes = []
    L.qm_gemm_mxfp4_bf16_nn.restype = i32
    L.qm_gemm_mxfp4_bf16_nn.argtypes = [vp, vp, vp, i64, i64, i64, f32, vp, i32, vp]
    L.qm_gemm_noalloc_prepare.restype = i32
    L.qm_gemm_noalloc_prepare.argtypes = []
    L.qm_gemm_fuses_rotation.restype = i32
    L.qm_gemm_fuses_rotation.argtypes = [vp, vp, i64, i64, i64]
    L.qm_gemm_mxfp4_tn_rotated.restype = i32
    L.qm_gemm_mxfp4_tn_rotated.argtypes = [vp, vp, vp, vp, i64, i64, i64, f32, vp, i32, i32, vp, vp, i32, vp]
    L.qm_gemm_mxfp4_tn_noalloc.restype = i32
    L.qm_gemm_mxfp4_tn_noalloc.argtypes = [vp, vp, vp, vp, i64, i64, i64, f32, vp, i32, i32, i32, vp]
    L.qm_masked_hadamard_bwd.restype = i32
    L.qm_masked_hadamard_bwd.argtypes = [vp, i32, i64, i64, i32, i32, vp, vp, vp, i32, vp]
    L.qm_dequantize_mxfp4.restype = i32
    L.qm_dequantize_mxfp4.argtypes = [vp, vp, i64, i64, f32, vp, i32, vp]
    sz = ctypes.c_size_t
    L.qm_packed_operand_bytes.restype = sz
    L.qm_packed_operand_bytes.argtypes = [i64, i64]
    L.qm_packed_operand_offsets.restype = i32
    L.qm_packed_operand_offsets.argtypes = [i64, i64, ctypes.POINTER(sz)]
    L.qm_linear_backward_workspace_bytes.restype = sz
    L.qm_linear_backward_workspace_bytes.argtypes = [i64, i64, i64, i32]
    L.qm_linear_forward.restype = i32
    L.qm_linear_forward.argtypes = [vp, i32, vp, i32, i64, i64, i64, i32, vp, i32, vp, vp, sz, vp, sz, i32, vp, i32, i32, vp]
    L.qm_rmsnorm_quantize_mxfp4.restype = i32
    L.qm_rmsnorm_quantize_mxfp4.argtypes = [vp, i32, vp, i32, vp, vp, f32, i64, i64, vp, vp, sz, vp, i32, vp]
    L.qm_swiglu_quantize_mxfp4.restype = i32
    L.qm_swiglu_quantize_mxfp4.argtypes = [vp, i32, i64, i64, vp, vp, sz, i32, vp]
    L.qm_rmsnorm_backward_workspace_bytes.restype = sz
    L.qm_rmsnorm_backward_workspace_bytes.argtypes = [i64, i64]
    L.qm_rmsnorm_backward.restype = i32
    L.qm_rmsnorm_backward.argtypes = [vp, i32, vp, i32, vp, vp, i64, i64, vp, vp, i32, vp, vp, vp, vp, vp, sz, vp]
    L.qm_swiglu_backward.restype = i32
    L.qm_swiglu_backward.argtypes = [vp, i32, vp, i32, i64, i64, vp, vp, i32, vp, vp]
    L.qm_rope_split_qkv.restype = i32
    L.qm_rope_split_qkv.argtypes = [vp, i32, i64, i64, i64, i32, vp, vp, vp, vp, i32, vp]
    L.qm_rope_merge_qkv_grad.restype = i32
    L.qm_rope_merge_qkv_grad.argtypes = [vp, vp, vp, i32, i64, i64, i64, i32, vp, vp, i32, vp]
    L.qm_linear_backward.restype = i32
    L.qm_linear_backward.argtypes = [vp, i32, i64, i64, i64, vp, vp, i32, vp, i32, vp, i32, vp, i32, vp, i32, i32, i32, i32, i32,
                                     vp, sz, vp, vp, i32, i32, i32, vp, vp]
    L.qm_linear_backward_seeded.restype = i32
    L.qm_linear_backward_seeded.argtypes = L.qm_linear_backward.argtypes[:-1] + [vp, vp]
    _lib = L
    return L


def check(rc, what):
    if rc != 0:
        msg = lib().qm_last_error().decode("utf-8", "replace")
        raise QuartetHipError(f"{what} failed (rc={rc}): {msg}")
