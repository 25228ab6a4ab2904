"""FP8 (e4m3fn) quantizer operators: the producers and consumers of the scale layouts the GEMMs use.
Each is one HIP launch through the C ABI on device tensors (group size 16 / 32 / 64 / 128; bf16 / f16 /
f32 activations; e4m3 codes).  There is no other path: host tensors and forms the kernels do not cover
raise.  Every quantizer clamps to +-448 before the cast and divides with IEEE division (x / scale),
as src/tilegym/suites/unsloth/cutile/fp8.py:105-116, the column-major kernel of
src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:78-145 and the reference's test
oracle of that operator do.  The reference's row-major kernel (per_token_group_quant_8bit.py:57-63)
multiplies by 1.0 / scale instead; its codes can differ from x / scale by one e4m3 code at rounding
boundaries, and the row-major form here follows the oracle's division, not that kernel."""

from __future__ import annotations

from typing import Tuple

import torch

from . import _lib

FP8 = torch.float8_e4m3fn
_GROUPS = (16, 32, 64, 128)
_ACT_DTYPES = (torch.bfloat16, torch.float16, torch.float32)


def _require_device(x: torch.Tensor, what: str, group: int) -> None:
    if not x.is_cuda:
        raise RuntimeError(f"{what}: needs a tensor on a HIP device, got one on {x.device}")
    if group not in _GROUPS:
        raise NotImplementedError(f"{what}: group size {group} is not implemented (supported: {_GROUPS})")
    if x.dtype not in _ACT_DTYPES:
        raise NotImplementedError(f"{what}: input dtype {x.dtype} is not implemented (bf16, f16, f32)")


def act_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token 1 x block_size quantization; all-zero block -> scale 1.0
    (src/tilegym/suites/unsloth/cutile/fp8.py:370-385)."""
    assert x.shape[-1] % block_size == 0, "last dim must be divisible by block_size"
    _require_device(x, "act_quant", block_size)
    return _lib.fp8_quant_group(x, block_size, 0.0, 0)


def per_token_group_quant_fp8(x: torch.Tensor, group_size: int = 128, eps: float = 1e-10,
                              scale_ue8m0: bool = False, column_major_scales: bool = False,
                              scale_tma_aligned: bool = False,
                              dst_dtype: torch.dtype = FP8) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per (token, group) quantization with amax clamped below by eps
    (src/tilegym/suites/flashinfer/cutile/per_token_group_quant_8bit.py:152-272); ``dst_dtype`` is
    float8_e4m3fn or int8 (scale = amax / 127, values clamped to [-128, 127] and converted toward zero, as the
    float -> int8 cast of the reference's oracle does).

    Scale layouts as there (:185-204): row-major ``x.shape[:-1] + (G,)``; ``column_major_scales``: a
    ``(tokens, G)`` tensor with strides ``(1, tokens)``; with ``scale_tma_aligned`` the reference fills a
    ``(G, ceil4(tokens))`` buffer and returns its first ``tokens`` columns transposed *and made contiguous*
    (:235-236), i.e. a row-major ``(tokens, G)`` tensor - which is written here directly.  The column-major
    forms are defined for 2-D ``x``.  ``scale_ue8m0`` rounds each scale up to a power of two (:127-131)."""
    assert x.shape[-1] % group_size == 0, "the last dimension of `x` must be divisible by `group_size`"
    assert x.is_contiguous(), "`x` must be contiguous"
    if scale_tma_aligned or scale_ue8m0:
        assert column_major_scales, "scale_tma_aligned or scale_ue8m0 requires column_major_scales=True"
    if dst_dtype not in (FP8, torch.int8):
        raise NotImplementedError(f"dst_dtype {dst_dtype} is not implemented (float8_e4m3fn, int8)")
    _require_device(x, "per_token_group_quant_8bit", group_size)
    groups = x.shape[-1] // group_size
    if column_major_scales and x.dim() != 2:
        raise NotImplementedError("column-major scales are implemented for 2-D inputs")
    scales = None
    if column_major_scales and not scale_tma_aligned:
        scales = torch.empty((groups, x.shape[0]), dtype=torch.float32, device=x.device).t()
    elif column_major_scales:
        scales = torch.empty((x.shape[0], groups), dtype=torch.float32, device=x.device)
    return _lib.fp8_quant_group(x, group_size, eps, 2 if scale_ue8m0 else 1, scales, dst_dtype)


def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128,
                   dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """y = fp8(x) * s[i // bs, j // bs]  (src/tilegym/suites/unsloth/cutile/fp8.py:348-367)."""
    assert x.dim() == 2 and s.dim() == 2
    if not x.is_cuda:
        raise RuntimeError(f"weight_dequant: needs a tensor on a HIP device, got one on {x.device}")
    if x.dtype != FP8 or dtype not in _ACT_DTYPES:
        raise NotImplementedError(f"weight_dequant: {x.dtype} -> {dtype} is not implemented (e4m3fn -> bf16 / f16 / f32)")
    return _lib.fp8_weight_dequant(x, s.float(), block_size, dtype)
