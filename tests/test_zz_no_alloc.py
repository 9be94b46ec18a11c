"""The allocation-free product entry point (qm_gemm_mxfp4_tn_noalloc) against qm_gemm_mxfp4_tn: same bits, on two calls
in a row that share the library's built-in scratch, the second on a smaller input; shapes beyond the scratch and bad
arguments are rejected."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _operands(M, N, K, seed, dev):
    g = torch.Generator().manual_seed(seed)
    mk = lambda r: (torch.randint(0, 256, (r, K // 2), generator=g, dtype=torch.uint8).to(dev),
                    torch.randint(118, 130, (r, K // 32), generator=g, dtype=torch.uint8).to(dev))
    return mk(M) + mk(N)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_noalloc_product_matches_the_allocating_entry_point(out_dtype):
    from quartet_amd import _lib, kernels as K
    dev = torch.device("cuda:0")
    L = _lib.lib()
    # both shapes are cut into K ranges (few tiles, long K), the second needs less scratch than the first
    shapes = [(512, 768, 8192), (256, 512, 4096)]
    assert L.qm_gemm_workspace_bytes(*shapes[0]) > L.qm_gemm_workspace_bytes(*shapes[1]) > 0
    for call, (M, N, Kd) in enumerate(shapes):
        print(f"case noalloc gemm call={call} shape={M}x{N}x{Kd} {out_dtype}", flush=True)
        ac, as_, bc, bs = _operands(M, N, Kd, 100 + call, dev)
        want = K.gemm_mxfp4_tn(ac, as_, bc, bs, 16.0 / 9.0, out_dtype)     # allocates its split-K workspace
        out = torch.full((M, N), float("nan"), dtype=out_dtype, device=dev)
        before = torch.cuda.memory_allocated()
        K.gemm_mxfp4_tn_noalloc(ac, as_, bc, bs, 16.0 / 9.0, out)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before
        assert torch.equal(out, want), f"call {call}: {(out.float() - want.float()).abs().max()}"
    # a shape without a split goes through as well (no scratch used)
    M, N, Kd = 512, 512, 512
    assert L.qm_gemm_workspace_bytes(M, N, Kd) == 0
    ac, as_, bc, bs = _operands(M, N, Kd, 7, dev)
    out = torch.empty((M, N), dtype=out_dtype, device=dev)
    assert torch.equal(K.gemm_mxfp4_tn_noalloc(ac, as_, bc, bs, 1.0, out), K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.0, out_dtype))


def test_noalloc_product_rejects_what_does_not_fit():
    from quartet_amd import _lib
    L = _lib.lib()
    cap = L.qm_gemm_noalloc_scratch_bytes()
    assert cap == 64 << 20
    M, N, Kd = 4096, 1536, 32768           # a weight-gradient shape whose partial sums exceed the built-in scratch
    assert L.qm_gemm_workspace_bytes(M, N, Kd) > cap
    # rejected before any pointer is touched
    assert L.qm_gemm_mxfp4_tn_noalloc(None, None, None, None, M, N, Kd, 1.0, None, 0, 0, 0, None) == -1
    assert b"built-in scratch" in L.qm_last_error()
    assert L.qm_gemm_mxfp4_tn_noalloc(None, None, None, None, 64, 64, 48, 1.0, None, 0, 0, 0, None) == -1
    assert L.qm_gemm_mxfp4_tn_noalloc(None, None, None, None, 0, 64, 64, 1.0, None, 0, 0, 0, None) == 0
