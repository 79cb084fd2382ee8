"""tp_gemm_static_ws -- the entry point for callers that cannot allocate -- against tp_gemm with a caller
workspace: the same plan and kernels, so the results are bit-identical.  Two calls in a row share the library's
built-in device array; the second is smaller and must not see anything the first left there."""
import ctypes

import pytest
import torch

DEV = "cuda:0"


def _desc(L, op, A, B, C, M, N, K, ksplit, epilogue=0, bias=None):
    from terapipe_amd import ops
    d = L.GemmDesc()
    d.op, d.dtype, d.epilogue = op, ops.tp_dtype(A.dtype), epilogue
    d.M, d.N, d.K = M, N, K
    d.A, d.lda = A.data_ptr(), A.stride(0)
    d.B, d.ldb = B.data_ptr(), B.stride(0)
    d.C, d.ldc = C.data_ptr(), C.stride(0)
    if bias is not None:
        d.bias = bias.data_ptr()
    d.reserved = ksplit << 8          # force the k split (bits 8-15), automatic tile configuration
    return d


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32], ids=str)
def test_static_workspace_gemm_matches_caller_workspace(dtype):
    from terapipe_amd import _lib as L
    lib = L.load(build_if_missing=False)
    g = torch.Generator(device=DEV).manual_seed(5)
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.tp_gemm_static_ws_capacity() == 64 << 20      # also looks up the array's address on this device
    # (op, M, N, K, k splits, epilogue): a large k-split product, then a smaller one with a bias epilogue, then one
    # whose plan does not split k at all (no workspace)
    cases = [(L.TP_GEMM_NT, 256, 2048, 8192, 4, L.TP_EPI_STORE),
             (L.TP_GEMM_NN, 96, 512, 4096, 3, L.TP_EPI_BIAS),
             (L.TP_GEMM_NT, 64, 256, 512, 1, L.TP_EPI_STORE)]
    for op, M, N, K, ks, epi in cases:
        A = (torch.randn(M, K, generator=g, device=DEV) * K ** -0.5).to(dtype)
        Bm = torch.randn((N, K) if op == L.TP_GEMM_NT else (K, N), generator=g, device=DEV).to(dtype)
        bias = torch.randn(N, generator=g, device=DEV).to(dtype)
        C0 = torch.full((M, N), 7.0, dtype=dtype, device=DEV)
        C1 = torch.full((M, N), 9.0, dtype=dtype, device=DEV)
        d0 = _desc(L, op, A, Bm, C0, M, N, K, ks, epi, bias)
        d1 = _desc(L, op, A, Bm, C1, M, N, K, ks, epi, bias)
        need = lib.tp_gemm_workspace_bytes(ctypes.byref(d0))
        assert need <= lib.tp_gemm_static_ws_capacity()
        if dtype != torch.float32:          # (the fp32 plan chooses its own k split)
            assert (need > 0) == (ks > 1)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
        print("static ws case op=%d %dx%dx%d splits=%d %s need=%d" % (op, M, N, K, ks, dtype, need), flush=True)
        L.check(lib.tp_gemm(ctypes.byref(d0), ws.data_ptr(), ws.numel(), stream), "tp_gemm")
        torch.cuda.synchronize()
        # the call under test allocates nothing: neither through torch nor behind its back (hipMemGetInfo)
        held, (free0, _) = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()
        L.check(lib.tp_gemm_static_ws(ctypes.byref(d1), stream), "tp_gemm_static_ws")
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == held
        assert torch.cuda.mem_get_info()[0] >= free0, "device memory shrank across tp_gemm_static_ws"
        assert torch.equal(C0, C1), "op %d %dx%dx%d" % (op, M, N, K)
        ref = A.double() @ (Bm.double().t() if op == L.TP_GEMM_NT else Bm.double())
        if epi == L.TP_EPI_BIAS:
            ref = ref + bias.double()
        err = ((C1.double() - ref).abs().max() / ref.abs().max()).item()
        assert err <= (1e-5 if dtype == torch.float32 else 2e-2), err


def test_static_workspace_entry_point_argument_errors_without_gpu(lib):
    """tp_gemm_static_ws: the capacity it states, and the refusals that need no GPU (a product whose k-split
    partial sums exceed the built-in array; defer_reduce, which would hand the array to a later call)."""
    from terapipe_amd import _lib
    cap = lib.tp_gemm_static_ws_capacity()
    assert cap == 64 << 20
    d = _lib.GemmDesc()
    assert lib.tp_gemm_static_ws(ctypes.byref(d), None) == 1                  # TP_ERR_ARG: empty descriptor
    d.op, d.dtype, d.epilogue = _lib.TP_GEMM_NT, _lib.TP_F16, _lib.TP_EPI_STORE
    d.M, d.N, d.K = 2048, 8192, 65536
    d.A = d.B = d.C = 256
    d.lda = d.ldb = d.K
    d.ldc = d.N
    d.reserved = 16 << 8                                                      # force 16 k splits
    need = lib.tp_gemm_workspace_bytes(ctypes.byref(d))
    assert need == 16 * 2048 * 8192 * 4 > cap
    assert lib.tp_gemm_static_ws(ctypes.byref(d), None) == 3                  # TP_ERR_WORKSPACE
    assert b"built-in" in lib.tp_last_error()
    d.reserved = 0
    d.defer_reduce = 1
    assert lib.tp_gemm_static_ws(ctypes.byref(d), None) == 1
    assert b"defer_reduce" in lib.tp_last_error()
