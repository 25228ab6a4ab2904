"""Stubs with the reference's signatures (src/tilegym/suites/unsloth/ops.py:199-265)."""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from ... import quant as _quant
from ...backend import dispatch, get_current_backend, register_impl
from ...ops import hip as _hip  # noqa: F401  (registers unsloth.w8a8_block_fp8_matmul)


@dispatch("unsloth.weight_dequant")
def weight_dequant(x: torch.Tensor, s: torch.Tensor, block_size: int = 128,
                   dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """FP8 block-wise weight dequantization: x (M,N) fp8, s (ceil(M/bs), ceil(N/bs))."""
    raise NotImplementedError(f"weight_dequant not implemented for {get_current_backend()}")


@dispatch("unsloth.act_quant")
def act_quant(x: torch.Tensor, block_size: int = 128) -> Tuple[torch.Tensor, torch.Tensor]:
    """FP8 block-wise activation quantization -> (y fp8, s per-block scales)."""
    raise NotImplementedError(f"act_quant not implemented for {get_current_backend()}")


@dispatch("unsloth.w8a8_block_fp8_matmul")
def w8a8_block_fp8_matmul(A: torch.Tensor, B: torch.Tensor, As: torch.Tensor, Bs: torch.Tensor,
                          block_size: Optional[List[int]] = None,
                          output_dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """Block-wise FP8 matmul (W8A8): A (...,K) fp8, B (N,K) fp8, As (..., ceil(K/bk)),
    Bs (ceil(N/bn), ceil(K/bk)); returns (..., N)."""
    raise NotImplementedError(f"w8a8_block_fp8_matmul not implemented for {get_current_backend()}")


register_impl("unsloth.weight_dequant", backend="hip")(_quant.weight_dequant)
register_impl("unsloth.act_quant", backend="hip")(_quant.act_quant)
