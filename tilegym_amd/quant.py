"""FP8 (e4m3fn) quantizers: the producers of the scale layouts the GEMMs consume.  The per-token
1 x 128 activation quantizers run as one HIP launch for device tensors (bf16 / f16 / f32,
group size 128); the other forms, and host tensors (synthetic workload generation), use the same
arithmetic in torch ops.  Every quantizer clamps to +-448 before the cast (torch's cast does not
saturate) and divides with IEEE division, as the reference's kernels do
(src/tilegym/suites/unsloth/cutile/fp8.py:105-116,
src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:52-66)."""

from __future__ import annotations

from typing import Optional, Tuple

import torch

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0


def _hip_1x128_ok(x: torch.Tensor, group: int) -> bool:
    return (x.is_cuda and group == 128 and x.numel() > 0 and x.dtype in (torch.bfloat16, torch.float16, torch.float32)
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
    if _hip_1x128_ok(x, block_size):
        from . import _lib
        return _lib.fp8_quant_1x128(x, 0.0, False)
    xb = x.contiguous().float().reshape(-1, block_size)
    amax = xb.abs().amax(dim=-1, keepdim=True)
    s = amax / FP8_MAX
    s = torch.where(s == 0, torch.ones_like(s), s)
    q = (xb / s).clamp(-FP8_MAX, FP8_MAX).to(FP8).reshape(x.shape)
    return q, s.reshape(*x.shape[:-1], x.shape[-1] // block_size)


def per_token_group_quant_fp8(x: torch.Tensor, group_size: int = 128, eps: float = 1e-10,
                              scale_ue8m0: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per (token, group) quantization with amax clamped below by eps, row-major scales
    (src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:152-272)."""
    assert x.shape[-1] % group_size == 0 and x.is_contiguous()
    if not scale_ue8m0 and _hip_1x128_ok(x, group_size):
        from . import _lib
        return _lib.fp8_quant_1x128(x, eps, True)
    xb = x.float().reshape(-1, group_size)
    amax = xb.abs().amax(dim=-1, keepdim=True).clamp(min=eps)
    s = amax / FP8_MAX
    if scale_ue8m0:
        s = torch.exp2(torch.ceil(torch.log2(s.abs().clamp(min=1e-10))))
    q = (xb / s).clamp(-FP8_MAX, FP8_MAX).to(FP8).reshape(x.shape)
    return q, s.reshape(*x.shape[:-1], x.shape[-1] // group_size)


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
    M, N = x.shape
    se = s.repeat_interleave(block_size, 0)[:M].repeat_interleave(block_size, 1)[:, :N]
    return (x.float() * se).to(dtype)
