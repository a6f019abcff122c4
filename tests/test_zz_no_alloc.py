"""cs_gemm_rmsnorm_noalloc: the RMSNorm-folded GEMM whose row-sums workspace is a static device array of the library,
against the same two launches with a caller-allocated workspace (cs_row_sumsq + cs_gemm), through the C ABI."""

import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _args(lib, a, w, bias, out, epilogue, eps, sums=None):
    g = lib.CsGemmArgs()
    g.A, g.lda = a.data_ptr(), a.stride(0)
    g.W, g.ldw = w.data_ptr(), w.stride(0)
    g.bias = bias.data_ptr()
    g.C, g.ldc = out.data_ptr(), out.stride(0)
    g.M, g.N, g.K = a.shape[0], w.shape[0], a.shape[1]
    g.epilogue = epilogue
    g.norm_eps = eps
    g.a_row_sumsq = None if sums is None else sums.data_ptr()
    return g


def test_no_alloc_entry_point_equals_the_workspace_form():
    from cornserve_amd import lib

    dll = lib.load()
    dev = torch.device("cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    gen = torch.Generator().manual_seed(7)
    # two calls in a row on the one static array, the second smaller in both rows and normalised width (so that it
    # leaves parts of the first call's sums behind in the array, which it must not read)
    for M, N, K, epi in ((8192, 3840, 1280, lib.EPI_BIAS), (1000, 2304, 320, lib.EPI_SWIGLU)):
        a = (torch.randn((M, K), generator=gen) * 2.0).bfloat16().to(dev)
        w = (torch.randn((N, K), generator=gen) * 0.05).bfloat16().to(dev)
        b = (torch.randn((N,), generator=gen) * 0.02).bfloat16().to(dev)
        n_out = N // 2 if epi == lib.EPI_SWIGLU else N
        # the existing entry points with a caller-allocated workspace
        sums = torch.full((M, 8), 3.0, dtype=torch.float32, device=dev)
        want = torch.zeros((M, n_out), dtype=torch.bfloat16, device=dev)
        lib.check(dll.cs_row_sumsq(a.data_ptr(), a.stride(0), M, K, sums.data_ptr(), stream), "cs_row_sumsq")
        lib.check(dll.cs_gemm(ctypes.byref(_args(lib, a, w, b, want, epi, 1e-6, sums)), stream), "cs_gemm")
        # the entry point that allocates nothing
        got = torch.zeros((M, n_out), dtype=torch.bfloat16, device=dev)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(dev)
        lib.check(dll.cs_gemm_rmsnorm_noalloc(ctypes.byref(_args(lib, a, w, b, got, epi, 1e-6)), stream),
                  "cs_gemm_rmsnorm_noalloc")
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(dev) == before
        assert torch.equal(got, want), (M, N, K)
        # and the result is the normalised product (fp32 reference on a sample of rows)
        rows = torch.arange(0, M, 97)
        af = a.float().cpu()[rows]
        ref = (af * torch.rsqrt(af.pow(2).mean(-1, keepdim=True) + 1e-6)) @ w.float().cpu().t() + b.float().cpu()
        if epi == lib.EPI_SWIGLU:
            ref = torch.nn.functional.silu(ref[:, 0::2].bfloat16().float()) * ref[:, 1::2].bfloat16().float()
        err = (got.float().cpu()[rows] - ref).abs().max().item()
        assert err <= 2.0**-7 * ref.abs().max().item(), err

    # sizes beyond the static array are refused, and so is a caller-supplied workspace
    big = lib.CsGemmArgs()
    big.A, big.W, big.C = a.data_ptr(), w.data_ptr(), got.data_ptr()
    big.lda = big.ldw = K
    big.ldc = N
    big.M, big.N, big.K = 65537, N, K
    assert dll.cs_gemm_rmsnorm_noalloc(ctypes.byref(big), stream) == lib.CS_ERR_TOO_LARGE
    wide = _args(lib, a, w, b, got, lib.EPI_BIAS, 1e-6)
    wide.K = 1288
    assert dll.cs_gemm_rmsnorm_noalloc(ctypes.byref(wide), stream) == lib.CS_ERR_TOO_LARGE
    own = _args(lib, a, w, b, got, lib.EPI_BIAS, 1e-6, sums)
    assert dll.cs_gemm_rmsnorm_noalloc(ctypes.byref(own), stream) == lib.CS_ERR_INVALID_ARG
    # shapes and epilogues the folded form does not exist for are refused before anything is enqueued
    odd_k = _args(lib, a, w, b, got, lib.EPI_BIAS, 1e-6)
    odd_k.K = 296
    assert dll.cs_gemm_rmsnorm_noalloc(ctypes.byref(odd_k), stream) == lib.CS_ERR_UNSUPPORTED
    short_k = _args(lib, a, w, b, got, lib.EPI_BIAS, 1e-6)
    short_k.K = 128
    assert dll.cs_gemm_rmsnorm_noalloc(ctypes.byref(short_k), stream) == lib.CS_ERR_UNSUPPORTED
    gelu = _args(lib, a, w, b, got, lib.EPI_GELU_ERF, 1e-6)
    assert dll.cs_gemm_rmsnorm_noalloc(ctypes.byref(gelu), stream) == lib.CS_ERR_UNSUPPORTED
    torch.cuda.synchronize()
