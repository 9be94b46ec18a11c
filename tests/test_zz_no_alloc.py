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
        K.gemm_noalloc_prepare()      # the one step that may load the library's device image; a no-op from then on
        torch.cuda.synchronize()
        # free device memory as the driver reports it (hipMemGetInfo): it sees allocations of the library and of the HIP
        # runtime as well, which torch's own allocator statistics would not
        before, before_torch = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
        K.gemm_mxfp4_tn_noalloc(ac, as_, bc, bs, 16.0 / 9.0, out)
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == before and torch.cuda.memory_allocated() == before_torch
        assert torch.equal(out, want), f"call {call}: {(out.float() - want.float()).abs().max()}"
    # a shape without a split goes through as well (no scratch used)
    M, N, Kd = 512, 512, 512
    assert L.qm_gemm_workspace_bytes(M, N, Kd) == 0
    ac, as_, bc, bs = _operands(M, N, Kd, 7, dev)
    out = torch.empty((M, N), dtype=out_dtype, device=dev)
    assert torch.equal(K.gemm_mxfp4_tn_noalloc(ac, as_, bc, bs, 1.0, out), K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.0, out_dtype))


def test_noalloc_product_under_graph_capture():
    """A split-K product captured into a HIP graph through the allocation-free entry point: every replay, with eager work
    and synchronisations in between, gives the bits of the eager allocating call on the operands then in place."""
    from quartet_amd import _lib, kernels as K
    dev = torch.device("cuda:0")
    M, N, Kd = 512, 768, 8192
    assert _lib.lib().qm_gemm_workspace_bytes(M, N, Kd) > 0
    ac, as_, bc, bs = _operands(M, N, Kd, 300, dev)
    out = torch.zeros((M, N), dtype=torch.bfloat16, device=dev)
    K.gemm_noalloc_prepare()
    K.gemm_mxfp4_tn_noalloc(ac, as_, bc, bs, 1.0, out)        # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        K.gemm_mxfp4_tn_noalloc(ac, as_, bc, bs, 1.0, out)
    for replay in range(3):
        print(f"case noalloc gemm graph replay={replay}", flush=True)
        fresh = _operands(M, N, Kd, 310 + replay, dev)        # new operand bytes in the captured buffers
        for dst, src in zip((ac, as_, bc, bs), fresh):
            dst.copy_(src)
        want = K.gemm_mxfp4_tn(ac, as_, bc, bs, 1.0, torch.bfloat16)   # eager work between the replays (uses the stream)
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), f"replay {replay}"


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
