"""The residual add that allocates nothing (bw_gemm_add_bf16_static): called through ctypes, its
output must be the bits of bw_gemm_add_bf16 with a workspace from the caller, on two calls in a
row that share the library's static scratch, the second with a smaller input."""

import ctypes
from ctypes import c_int, c_longlong, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    from bitwise_amd.csrc import build

    lib = ctypes.CDLL(str(build.build()))      # the current library's path (nothing is compiled if it is there)
    lib.bw_gemm_add_bf16_static.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]
    lib.bw_gemm_add_bf16_static.restype = c_int
    lib.bw_gemm_add_bf16_static_max.argtypes = [c_void_p, c_void_p]
    lib.bw_gemm_add_bf16_static_max.restype = c_int
    lib.bw_gemm_add_scratch.argtypes = [c_int, c_int, c_int, c_void_p, c_void_p]
    lib.bw_gemm_add_scratch.restype = c_int
    lib.bw_gemm_add_bf16.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                     c_longlong, c_void_p, c_int, c_void_p]
    lib.bw_gemm_add_bf16.restype = c_int
    return lib


def _hip_runtime() -> ctypes.CDLL:
    """The HIP runtime this process has already loaded (the one torch and the kernel library call), by the path
    the process maps it from; a second copy of the runtime would count its own allocations only."""
    with open("/proc/self/maps") as f:
        paths = {line.split()[-1] for line in f if "libamdhip64.so" in line}
    assert len(paths) == 1, f"one HIP runtime is expected in the process, found {sorted(paths)}"
    return ctypes.CDLL(paths.pop())


def _free_device_memory() -> int:
    """Free bytes on the current device as the HIP runtime itself counts them: any hipMalloc or hipFree, by
    whomever, moves it; torch's own counters see only torch's allocator."""
    hip = _hip_runtime()
    hip.hipMemGetInfo.argtypes = [c_void_p, c_void_p]
    hip.hipMemGetInfo.restype = c_int
    free, total = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert hip.hipMemGetInfo(ctypes.addressof(free), ctypes.addressof(total)) == 0
    return free.value


def _scratch_need(lib, M, N, K):
    floats, counters = c_longlong(0), c_int(0)
    assert lib.bw_gemm_add_scratch(M, N, K, ctypes.addressof(floats), ctypes.addressof(counters)) == 0
    return floats.value, counters.value


def test_static_scratch_residual_add_matches_the_workspace_one(gpu):
    lib = _library()
    stream = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(11)
    # (rows, columns, inner size): both take the kernel whose segments of K meet in scratch; the second is smaller
    # in every size, so it finds the first call's sums and counters in the array
    for M, N, K in [(48, 2048, 8192), (20, 1024, 4096)]:
        floats, counters = _scratch_need(lib, M, N, K)
        assert floats > 0 and counters > 0, "this shape must be one that needs scratch"
        x = torch.randn(M, K, generator=g).to(torch.bfloat16).to(gpu)
        w = (torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).to(gpu)
        res = torch.randn(M, N, generator=g).to(gpu)
        want, got = res.clone(), res.clone()
        work = torch.zeros(floats, dtype=torch.float32, device=gpu)
        count = torch.zeros(counters, dtype=torch.int32, device=gpu)
        rc = lib.bw_gemm_add_bf16(x.data_ptr(), w.data_ptr(), want.data_ptr(), M, N, K, K, N, work.data_ptr(), floats,
                                  count.data_ptr(), counters, stream)
        assert rc == 0
        torch.cuda.synchronize()
        # a first call on a copy of the output (it may load the kernels' code and takes the array's address), then
        # the call that is measured: the runtime's free memory must not move, whoever might have allocated
        warm = res.clone()
        assert lib.bw_gemm_add_bf16_static(x.data_ptr(), w.data_ptr(), warm.data_ptr(), M, N, K, K, N, stream) == 0
        torch.cuda.synchronize()
        before, before_torch = _free_device_memory(), torch.cuda.memory_allocated(gpu)
        rc = lib.bw_gemm_add_bf16_static(x.data_ptr(), w.data_ptr(), got.data_ptr(), M, N, K, K, N, stream)
        assert rc == 0
        torch.cuda.synchronize()
        assert _free_device_memory() == before and torch.cuda.memory_allocated(gpu) == before_torch
        assert torch.equal(warm, got)
        assert not torch.equal(got, res), "the product must have been added"
        assert torch.equal(got.view(torch.int32), want.view(torch.int32)), (M, N, K)
        # and against the plain sum, so that two equal wrong results do not pass
        ref = res.double() + x.double() @ w.double().T
        assert (got.double() - ref).abs().max().item() < 2e-3 * max(1.0, ref.abs().max().item())


def test_the_free_memory_figure_sees_an_allocation(gpu):
    """The measure the test above relies on can fail: an allocation behind torch's back moves it."""
    hip = _hip_runtime()
    hip.hipMalloc.argtypes = [c_void_p, ctypes.c_size_t]
    hip.hipMalloc.restype = c_int
    hip.hipFree.argtypes = [c_void_p]
    hip.hipFree.restype = c_int
    torch.cuda.synchronize()
    before, before_torch = _free_device_memory(), torch.cuda.memory_allocated(gpu)
    ptr = c_void_p(0)
    assert hip.hipMalloc(ctypes.addressof(ptr), 64 << 20) == 0
    held = _free_device_memory()
    assert hip.hipFree(ptr) == 0
    assert held < before and torch.cuda.memory_allocated(gpu) == before_torch


def test_static_scratch_refuses_what_it_cannot_hold(gpu):
    lib = _library()
    stream = torch.cuda.current_stream().cuda_stream
    max_floats, max_counters = c_longlong(0), c_int(0)
    assert lib.bw_gemm_add_bf16_static_max(ctypes.addressof(max_floats), ctypes.addressof(max_counters)) == 0
    M, N, K = 64, 8192, 32768
    floats, _ = _scratch_need(lib, M, N, K)
    assert floats > max_floats.value
    x = torch.zeros(M, K, dtype=torch.bfloat16, device=gpu)
    w = torch.zeros(N, K, dtype=torch.bfloat16, device=gpu)
    out = torch.zeros(M, N, device=gpu)
    assert lib.bw_gemm_add_bf16_static(x.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K, K, N, stream) == -7
