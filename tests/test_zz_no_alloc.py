"""The entry point that allocates nothing, called through ctypes beside the entry point it is a variant of.

``vk_gemm_bf16_mid_no_alloc`` keeps the partial sums of a split-K product in a device array of the library
instead of a workspace the caller brings.  Two calls in a row, the second on a smaller input, must give the
outputs of ``vk_gemm_bf16_mid`` bit for bit: the second call finds the first one's partial sums in the array.
"""
import ctypes

import pytest
import torch

pytestmark = pytest.mark.gpu


def _library():
    import vipera_rs_amd  # noqa: F401
    from vipera_rs_amd.ops.build import library_path, load_module
    load_module("gemm_bf16")                       # builds it if nothing is built
    lib = ctypes.CDLL(library_path("gemm_bf16"))
    p, i, ll = ctypes.c_void_p, ctypes.c_int, ctypes.c_longlong
    lib.vk_gemm_bf16_mid.argtypes = [p, p, p, p, i, i, i, i, ll, ll, i, i, i, p, ll, p]
    lib.vk_gemm_bf16_mid.restype = i
    lib.vk_gemm_bf16_mid_no_alloc.argtypes = [p, p, p, p, i, i, i, i, ll, ll, i, i, i, p]
    lib.vk_gemm_bf16_mid_no_alloc.restype = i
    lib.vk_gemm_bf16_mid_no_alloc_capacity.restype = ll
    return lib


def _both(lib, m, n, k, ranges, seed, accumulate):
    device = torch.device("cuda:0")
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(m, k, generator=g).to(torch.bfloat16).to(device)
    w = (torch.randn(n, k, generator=g) * 0.05).to(torch.bfloat16).to(device)
    bias = torch.randn(n, generator=g).to(device)
    start = torch.randn(m, n, generator=g).to(device)
    workspace = torch.full((ranges * m * n,), float("nan"), device=device)
    outs = []
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for no_alloc in (False, True):
        out = start.clone()
        torch.cuda.synchronize()
        before = torch.cuda.memory_stats()["allocation.all.allocated"]
        common = (a.data_ptr(), w.data_ptr(), bias.data_ptr(), out.data_ptr(), 0, m, n, k, k, n,
                  1 if accumulate else 0, ranges, 1)
        if no_alloc:
            status = lib.vk_gemm_bf16_mid_no_alloc(*common, stream)
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == before
        else:
            status = lib.vk_gemm_bf16_mid(*common, workspace.data_ptr(), workspace.numel(), stream)
        assert status == 0, f"status {status}"
        torch.cuda.synchronize()
        outs.append(out)
    want = a.float() @ w.float().T + bias + (start if accumulate else 0)
    assert torch.allclose(outs[0], want, rtol=2e-2, atol=2e-2)      # the existing entry point is right,
    assert torch.equal(outs[0], outs[1])                            # and the new one equals it bit for bit
    return outs[1]


def test_two_calls_in_a_row_the_second_smaller():
    lib = _library()
    _both(lib, 48, 1000, 2048, 4, seed=1, accumulate=True)
    _both(lib, 5, 136, 512, 2, seed=2, accumulate=False)     # finds the larger call's partial sums in the array
    _both(lib, 64, 3584, 4096, 8, seed=3, accumulate=True)   # and a larger one again
    _both(lib, 100, 1000, 1544, 4, seed=4, accumulate=False)  # 65 to 128 tokens: the kernel's chunks of 128 along K
    _both(lib, 7, 200, 1024, 2, seed=5, accumulate=False)


def test_the_driver_sees_no_allocation_either():
    """Free device memory as the driver counts it (not torch's allocator, which a hipMalloc inside the library
    would pass by) is the same before and after a hundred calls, once the first call has run."""
    lib = _library()
    device = torch.device("cuda:0")
    m, n, k, ranges = 24, 1024, 2048, 4
    a = torch.randn(m, k).to(torch.bfloat16).to(device)
    w = (torch.randn(n, k) * 0.05).to(torch.bfloat16).to(device)
    out = torch.zeros(m, n, device=device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    args = (a.data_ptr(), w.data_ptr(), None, out.data_ptr(), 0, m, n, k, k, n, 0, ranges, 1, stream)
    assert lib.vk_gemm_bf16_mid_no_alloc(*args) == 0          # the first call on the device asks for the array's address
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    allocated_before = torch.cuda.memory_stats()["allocation.all.allocated"]
    for _ in range(100):
        assert lib.vk_gemm_bf16_mid_no_alloc(*args) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.cuda.memory_stats()["allocation.all.allocated"] == allocated_before
    assert torch.allclose(out, a.float() @ w.float().T, rtol=2e-2, atol=2e-2)


def test_sizes_beyond_the_array_are_refused():
    lib = _library()
    capacity = lib.vk_gemm_bf16_mid_no_alloc_capacity()
    assert capacity == 4 * 1024 * 1024
    device = torch.device("cuda:0")
    m, k, ranges = 64, 64, 16
    n = capacity // (ranges * m) + 8
    a = torch.zeros(m, k, dtype=torch.bfloat16, device=device)
    w = torch.zeros(n, k, dtype=torch.bfloat16, device=device)
    out = torch.zeros(m, n, device=device)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    status = lib.vk_gemm_bf16_mid_no_alloc(a.data_ptr(), w.data_ptr(), None, out.data_ptr(), 0, m, n, k, k, n, 0, ranges,
                                           1, stream)
    assert status == -2
    # sizes whose product would not fit 64 bits do not slip past the check either
    assert lib.vk_gemm_bf16_mid_no_alloc(a.data_ptr(), w.data_ptr(), None, out.data_ptr(), 0, 2 ** 31 - 1, 2 ** 31 - 1, k,
                                         k, n, 0, 2 ** 31 - 1, 1, stream) == -2
    torch.cuda.synchronize()
    assert not out.any()
