"""Stubs with the reference's signatures (src/tilegym/suites/flashinfer/ops.py:25-55,123-158,453-468)."""

from __future__ import annotations

from typing import Tuple

import torch

from ... import quant as _quant
from ...backend import dispatch, get_current_backend, register_impl
from ...ops import hip as _hip  # noqa: F401  (registers the flashinfer.gemm.* implementations)


@dispatch("flashinfer.gemm.gemm_alpha_beta")
def gemm_alpha_beta(a: torch.Tensor, b: torch.Tensor, c: torch.Tensor, trans_a: bool = False,
                    trans_b: bool = True, alpha: float = 1.0, beta: float = 0.0, num_sms: int = 1):
    """C = alpha * A @ B + beta * C, in place; returns C."""
    raise NotImplementedError(f"flashinfer.gemm.gemm_alpha_beta is not implemented for {get_current_backend()}")


@dispatch("flashinfer.gemm.ragged_block_scaled_bmm")
def ragged_block_scaled_bmm(a: torch.Tensor, b: torch.Tensor, a_scale: torch.Tensor,
                            b_scale: torch.Tensor, m_indptr: torch.Tensor, max_m: int,
                            max_m_device: torch.Tensor = None, transpose_a: bool = False,
                            transpose_b: bool = True, out_dtype: torch.dtype = None):
    """Ragged batched GEMM with block scales: a (total_m,K), b (Q,N,K), m_indptr (Q+1) ->
    c (total_m,N)."""
    raise NotImplementedError(f"flashinfer.gemm.ragged_block_scaled_bmm is not implemented for {get_current_backend()}")


@dispatch("flashinfer.per_token_group_quant_8bit")
def per_token_group_quant_8bit(x: torch.Tensor, group_size: int, eps: float = 1e-10,
                               dst_dtype: torch.dtype = torch.float8_e4m3fn,
                               column_major_scales: bool = False, scale_tma_aligned: bool = False,
                               scale_ue8m0: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Per-token-group 8-bit quantization -> (x_q, x_s)."""
    raise NotImplementedError(f"per_token_group_quant_8bit is not implemented for {get_current_backend()}")


@register_impl("flashinfer.per_token_group_quant_8bit", backend="hip")
def _per_token_group_quant_8bit(x, group_size, eps=1e-10, dst_dtype=torch.float8_e4m3fn,
                                column_major_scales=False, scale_tma_aligned=False, scale_ue8m0=False):
    if dst_dtype is None:
        dst_dtype = torch.float8_e4m3fn
    return _quant.per_token_group_quant_fp8(x, group_size, eps, scale_ue8m0, column_major_scales, scale_tma_aligned, dst_dtype)
