"""MoE entry points with the reference's signatures (src/tilegym/ops/moe_interface.py:14-79)."""

from __future__ import annotations

from typing import Any, Dict, Optional, Tuple

import torch

from ..backend import dispatch, get_current_backend


@dispatch("invoke_fused_moe_kernel")
def invoke_fused_moe_kernel(
    A: torch.Tensor,
    B: torch.Tensor,
    C: torch.Tensor,
    A_scale: Optional[torch.Tensor],
    B_scale: Optional[torch.Tensor],
    topk_weights: torch.Tensor,
    topk_ids: torch.Tensor,
    sorted_token_ids: torch.Tensor,
    expert_ids: torch.Tensor,
    num_tokens_post_padded: torch.Tensor,
    mul_routed_weight: bool,
    top_k: int,
    config: Dict[str, Any],
    compute_type: Any = None,
    use_fp8_w8a8: bool = True,
    use_int8_w8a16: bool = False,
    block_shape: Optional[list] = None,
) -> None:
    """Token-gather MoE GEMM; writes C (T, top_k, N) in place and returns None
    (src/tilegym/ops/moe_interface.py:14-18, src/tilegym/ops/tilecpp/moe.py:241-310)."""
    raise NotImplementedError(f"invoke_fused_moe_kernel is not implemented for {get_current_backend()}")


@dispatch("moe_align_block_size")
def moe_align_block_size(
    topk_ids: torch.Tensor, block_size: int, num_experts: int
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Sort (token, k) slots by expert and pad every expert to a multiple of block_size
    (src/tilegym/ops/moe_interface.py:21-28, src/tilegym/ops/cutile/moe_align_block.py:205-268)."""
    raise NotImplementedError(f"moe_align_block_size is not implemented for this backend: {get_current_backend()}")
