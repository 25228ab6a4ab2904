"""FP8 (e4m3fn) quantizers: the producers of the scale layouts the GEMMs consume.  The per-token
group activation quantizers (group size 16 / 32 / 64 / 128; bf16 / f16 / f32) and the weight
dequantizer run as one HIP launch for device tensors; other group sizes, and host tensors (synthetic
workload generation), use the same arithmetic in torch ops.  Every quantizer clamps to +-448 before the cast (torch's cast does not
saturate) and divides with IEEE division, as the reference's kernels do
(src/tilegym/suites/unsloth/cutile/fp8.py:105-116,
src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:52-66)."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


_HIP_GROUPS = (16, 32, 64, 128)


def _hip_group_ok(x: torch.Tensor, group: int) -> bool:
    return (x.is_cuda and group in _HIP_GROUPS and x.numel() > 0 and x.dtype in (torch.bfloat16, torch.float16, torch.float32)
            and x.data_ptr() % 16 == 0)


def quantize_per_tensor(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """One fp32 scale for the whole tensor: scale = amax/448 (1.0 for an all-zero tensor)."""
    xf = x.float()
    amax = xf.abs().amax()
    scale = torch.where(amax == 0, torch.ones_like(amax), amax / FP8_MAX)
    q = (xf / scale).clamp(-FP8_MAX, FP8_MAX).to(FP8)
    return q, scale.reshape(1)


def act_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token 1 x block_size quantization; all-zero block -> scale 1.0
    (src/tilegym/suites/unsloth/cutile/fp8.py:370-385)."""
    assert x.shape[-1] % block_size == 0, "last dim must be divisible by block_size"
    if _hip_group_ok(x, block_size):
        from . import _lib
        return _lib.fp8_quant_group(x, block_size, 0.0, 0)
    xb = x.contiguous().float().reshape(-1, block_size)
    amax = xb.abs().amax(dim=-1, keepdim=True)
    s = amax / FP8_MAX
    s = torch.where(s == 0, torch.ones_like(s), s)
    q = (xb / s).clamp(-FP8_MAX, FP8_MAX).to(FP8).reshape(x.shape)
    return q, s.reshape(*x.shape[:-1], x.shape[-1] // block_size)


def per_token_group_quant_fp8(x: torch.Tensor, group_size: int = 128, eps: float = 1e-10,
                              scale_ue8m0: bool = False, column_major_scales: bool = False,
                              scale_tma_aligned: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per (token, group) quantization with amax clamped below by eps
    (src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:152-272).

    Scale layouts as there (:185-204): row-major ``x.shape[:-1] + (G,)``; ``column_major_scales``: a
    ``(tokens, G)`` tensor with strides ``(1, tokens)``; with ``scale_tma_aligned`` the reference fills a
    ``(G, ceil4(tokens))`` buffer and returns its first ``tokens`` columns transposed *and made contiguous*
    (:235-236), i.e. a row-major ``(tokens, G)`` tensor - which is written here directly.  The column-major
    forms are defined for 2-D ``x``.  ``scale_ue8m0`` rounds each scale up to a power of two (:127-131)."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` must be divisible by `group_size`"
    assert x.is_contiguous(), "`x` must be contiguous"
    if scale_tma_aligned or scale_ue8m0:
        assert column_major_scales, "scale_tma_aligned or scale_ue8m0 requires column_major_scales=True"
    groups = x.shape[-1] // group_size
    if column_major_scales and x.dim() != 2:
        raise NotImplementedError("column-major scales are implemented for 2-D inputs")
    if _hip_group_ok(x, group_size):
        from . import _lib
        scales = None
        if column_major_scales and not scale_tma_aligned:
            scales = torch.empty((groups, x.shape[0]), dtype=torch.float32, device=x.device).t()
        elif column_major_scales:
            scales = torch.empty((x.shape[0], groups), dtype=torch.float32, device=x.device)
        return _lib.fp8_quant_group(x, group_size, eps, 2 if scale_ue8m0 else 1, scales)
    xb = x.float().reshape(-1, group_size)
    amax = xb.abs().amax(dim=-1, keepdim=True).clamp(min=eps)
    s = amax / FP8_MAX
    if scale_ue8m0:
        s = torch.exp2(torch.ceil(torch.log2(s.abs().clamp(min=1e-10))))
    q = (xb / s).clamp(-FP8_MAX, FP8_MAX).to(FP8).reshape(x.shape)
    s = s.reshape(*x.shape[:-1], groups)
    if column_major_scales and not scale_tma_aligned:
        s = s.t().contiguous().t()
    return q, s


def weight_quant_block(w: torch.Tensor, block_n: int = 128, block_k: int = 128):
    """Per (block_n x block_k) block quantization of a (N, K) weight -> (q, Bs (ceil(N/bn), ceil(K/bk)))."""
    N, K = w.shape
    nb, kb = -(-N // block_n), -(-K // block_k)
    wp = torch.zeros(nb * block_n, kb * block_k, dtype=torch.float32, device=w.device)
    wp[:N, :K] = w.float()
    blocks = wp.reshape(nb, block_n, kb, block_k)
    amax = blocks.abs().amax(dim=(1, 3))
    s = torch.where(amax == 0, torch.ones_like(amax), amax / FP8_MAX)
    q = (blocks / s[:, None, :, None]).clamp(-FP8_MAX, FP8_MAX)
    q = q.reshape(nb * block_n, kb * block_k)[:N, :K].contiguous().to(FP8)
    return q, s


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128,
                   dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """y = fp8(x) * s[i // bs, j // bs]  (src/tilegym/suites/unsloth/cutile/fp8.py:348-367)."""
    assert x.dim() == 2 and s.dim() == 2
    if x.is_cuda and x.numel() > 0 and x.dtype == FP8 and dtype in (torch.bfloat16, torch.float16, torch.float32):
        from . import _lib
        return _lib.fp8_weight_dequant(x, s.float(), block_size, dtype)
    M, N = x.shape
    se = s.repeat_interleave(block_size, 0)[:M].repeat_interleave(block_size, 1)[:, :N]
    return (x.float() * se).to(dtype)
