"""tg_fp8_gemm_static_scratch (the entry point for callers that cannot allocate) against tg_fp8_gemm.

Both are called through the C ABI on the same device tensors; integer work inside (fixed reduction order), so
the outputs must agree bit for bit.  Two calls in a row, the second on a smaller problem: the scratch array is
shared by every call on the GPU and keeps the previous call's contents."""

import pytest
import torch

from tilegym_amd import _lib

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn


def _case(M, N, K, seed, device, trans_b=True):
    g = torch.Generator().manual_seed(seed)
    a = torch.randn(M, K, generator=g).clamp(-448, 448).to(FP8).to(device)
    shape = (N, K) if trans_b else (K, N)
    b = (torch.randn(shape, generator=g) * 0.05).to(FP8).to(device)
    sa = torch.tensor([0.5], device=device)
    sb = torch.tensor([1.25], device=device)
    return a, b, sa, sb


def _both(a, b, sa, sb, M, N, trans_b=True, kernel_configs=None):
    c_ref = torch.zeros(M, N, dtype=torch.bfloat16, device=a.device)
    c_new = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=a.device)
    _lib.fp8_gemm(c_ref, a, b, sa, sb, trans_b=trans_b, kernel_configs=kernel_configs)
    want = _lib.last_config()
    _lib.fp8_gemm_static_scratch(c_new, a, b, sa, sb, trans_b=trans_b, kernel_configs=kernel_configs)
    got = _lib.last_config()
    assert got == want, f"schedules differ: {got} vs {want}"
    torch.cuda.synchronize()
    return c_ref, c_new, got


def test_static_scratch_matches_workspace_form_twice(device):
    # first call: decode-sized down projection, split-K partial sums go through the scratch array
    M, N, K = 16, 4096, 14336
    a, b, sa, sb = _case(M, N, K, 1, device)
    c_ref, c_new, cfg = _both(a, b, sa, sb, M, N)
    assert cfg["SPLIT_K"] > 1, cfg
    assert torch.equal(c_ref, c_new)
    # second call, smaller problem, split-K forced: must not see the first call's partial sums
    M2, N2, K2 = 5, 328, 2048
    a2, b2, sa2, sb2 = _case(M2, N2, K2, 2, device)
    c_ref2, c_new2, cfg2 = _both(a2, b2, sa2, sb2, M2, N2, kernel_configs={"SPLIT_K": 4})
    assert cfg2["SPLIT_K"] > 1, cfg2
    assert torch.equal(c_ref2, c_new2)
    # and a mid-size one on the tiled kernel with split-K, then a (K,N) weight (its copy lives in the scratch too)
    M3, N3, K3 = 200, 264, 2048
    a3, b3, sa3, sb3 = _case(M3, N3, K3, 3, device)
    c_ref3, c_new3, cfg3 = _both(a3, b3, sa3, sb3, M3, N3, kernel_configs={"KERNEL": "tiled", "BLOCK_M": 128, "BLOCK_N": 128, "SPLIT_K": 3})
    assert cfg3["SPLIT_K"] > 1 and torch.equal(c_ref3, c_new3)
    a4, b4, sa4, sb4 = _case(64, 512, 1024, 4, device, trans_b=False)
    c_ref4, c_new4, _ = _both(a4, b4, sa4, sb4, 64, 512, trans_b=False)
    assert torch.equal(c_ref4, c_new4)


def test_static_scratch_rejects_what_does_not_fit(device):
    # (K,N) weight of 64 MiB: its K-contiguous copy does not fit the 32 MiB array
    M, N, K = 16, 8192, 8192
    a, b, sa, sb = _case(M, N, K, 5, device, trans_b=False)
    c = torch.empty(M, N, dtype=torch.bfloat16, device=device)
    with pytest.raises(_lib.TileGymHipError) as ei:
        _lib.fp8_gemm_static_scratch(c, a, b, sa, sb, trans_b=False)
    assert ei.value.rc == -6 and "static scratch" in str(ei.value)
    # split-K partial sums beyond the array: 8 x 2048 x 1024 x 4 bytes = 64 MiB
    a, b, sa, sb = _case(2048, 1024, 4096, 6, device)
    c = torch.empty(2048, 1024, dtype=torch.bfloat16, device=device)
    with pytest.raises(_lib.TileGymHipError) as ei:
        _lib.fp8_gemm_static_scratch(c, a, b, sa, sb, kernel_configs={"KERNEL": "tiled", "BLOCK_M": 128, "BLOCK_N": 128, "SPLIT_K": 8})
    assert ei.value.rc == -6 and "static scratch" in str(ei.value)


def test_static_scratch_allocates_nothing(device):
    M, N, K = 16, 4096, 14336
    a, b, sa, sb = _case(M, N, K, 7, device)
    c = torch.empty(M, N, dtype=torch.bfloat16, device=device)
    _lib.fp8_gemm_static_scratch(c, a, b, sa, sb)  # first call on the device: looks the array up
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    res0 = torch.cuda.memory_reserved()
    for _ in range(5):
        _lib.fp8_gemm_static_scratch(c, a, b, sa, sb)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert torch.cuda.memory_reserved() == res0 and free1 == free0
