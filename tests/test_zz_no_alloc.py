"""The GEMM entry point that allocates nothing (``ttbfp_gemm_bfp8b_bf16_static``): its workspace is a static device
array inside the library.  It runs the kernels of ``ttbfp_gemm_bfp8b_bf16_ws``, so on the same inputs the two must
agree bit for bit - checked on calls in a row that share the array (a larger split over K, a smaller one that leaves
most of the array as the first call filled it, a bf16 panel), with the driver's count of free device memory (which sees
a hipMalloc made anywhere in the process, the library included) and torch's allocator watched for any request."""
import ctypes
import sys

import pytest
import torch

from tt_buda_amd import capi

pytestmark = pytest.mark.gpu

F = capi.DataFormatCode
DEV = "cuda:0"


def say(*a):
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def gemm_static(x, wp, N, bias, epilogue, out):
    M, K = x.shape
    capi.check(capi.lib().ttbfp_gemm_bfp8b_bf16_static(M, N, K, x.data_ptr(), wp.data_ptr(), bias.data_ptr() if bias is not None else None,
                                                      epilogue, out.data_ptr(), capi._TORCH_FMT[out.dtype],
                                                      ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    return out


def case(M, N, K, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    w = torch.randn(1, 1, K, N, generator=g, device=DEV) * 0.02
    x = torch.randn(M, K, generator=g, device=DEV).bfloat16()
    bias = (torch.randn(N, generator=g, device=DEV) * 0.02).bfloat16()
    return x, capi.tilize_pack(w, F.Bfp8_b), bias


def test_static_scratch_gemm_matches_the_workspace_form_call_after_call():
    capi.check(capi.lib().ttbfp_init(0))
    limit = capi.lib().ttbfp_static_scratch_bytes()
    assert limit == 64 << 20
    # (M, N, K): split over K with 16 MiB of partial planes; a smaller split (8 MiB) right after it; a bf16 panel (24 MiB);
    # a shape that uses no workspace at all
    shapes = [(256, 4096, 4096), (256, 1024, 4096), (4096, 3072, 4096), (128, 1024, 1024)]
    for i, (M, N, K) in enumerate(shapes):
        need = capi.gemm_workspace_bytes(M, N, K)
        say("static scratch gemm", (M, N, K), "workspace bytes", need)
        assert need <= limit and (need > 0 or i == 3)
        x, wp, bias = case(M, N, K, 100 + i)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
        for out_dtype, epi, b in ((torch.bfloat16, capi.EPILOGUE_NONE, None), (torch.float32, capi.EPILOGUE_GELU, bias)):
            want = capi.gemm_bfp8b(x, wp, N, bias=b, epilogue=epi, out_dtype=out_dtype, workspace=ws)
            got = torch.full((M, N), float("nan"), dtype=out_dtype, device=DEV)
            gemm_static(x, wp, N, b, epi, got)  # warm-up: the kernels' code objects and attributes are set up once
            torch.cuda.synchronize()
            before = torch.cuda.memory_stats()["allocation.all.allocated"]
            free_before = torch.cuda.mem_get_info()[0]  # hipMemGetInfo: device memory free, whoever allocated the rest
            gemm_static(x, wp, N, b, epi, got)
            gemm_static(x, wp, N, b, epi, got)  # again on the array as the first call left it
            free_during = torch.cuda.mem_get_info()[0]  # the calls have been queued, nothing has been freed yet
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before == free_during, "device memory was allocated or freed during the calls"
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
            assert torch.equal(got, want), (M, N, K, out_dtype)


def test_static_scratch_gemm_refuses_what_does_not_fit():
    M = N = K = 8192  # the panel of this shape is 128 MiB
    assert capi.gemm_workspace_bytes(M, N, K) > capi.lib().ttbfp_static_scratch_bytes()
    x = torch.zeros(M, K, dtype=torch.bfloat16, device=DEV)
    wp = torch.zeros(capi.packed_size(F.Bfp8_b, (1, 1, K, N)), dtype=torch.uint8, device=DEV)
    y = torch.zeros(M, N, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(capi.BackendError) as ei:
        gemm_static(x, wp, N, None, capi.EPILOGUE_NONE, y)
    assert ei.value.status == capi.RUNTIME_ERROR and "static scratch holds" in str(ei.value)
    assert not y.any()
