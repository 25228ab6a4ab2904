"""The HIP FP8 GEMM entry points as operators of torch's dispatcher: ``torch.ops.tilegym_hip.*``.

The reference launches its kernels from Python on torch's current stream
(src/tilegym/ops/cutile/matmul.py:446-455); callers that key on torch's dispatcher -- ``torch.compile`` graphs,
``torch.library.opcheck``, anything that enumerates ``torch.ops`` -- cannot see a plain Python function.  Each operator
below is a thin ``torch.library.custom_op`` over the same C-ABI call the ``tilegym_amd.ops`` functions make (one
implementation, two ways in), with a shape-only "fake" implementation so that a graph can be traced without a GPU.
They are registered for device tensors only: with CPU tensors the dispatcher raises (there is no CPU implementation).

    fp8_gemm(a, b, scale_a, scale_b, trans_a, trans_b, alpha, out_dtype) -> c          tg_fp8_gemm
    fp8_gemm_out(c, a, b, scale_a, scale_b, trans_a, trans_b, alpha, beta) -> ()       tg_fp8_gemm, in place
    fp8_ragged_gemm(a, b, a_scale, b_scale, m_indptr, out_dtype) -> c                  tg_fp8_ragged_gemm
    fp8_moe_gemm_out(c, a, b, a_scale, b_scale, topk_weights, sorted_token_ids, expert_ids,
                     num_tokens_post_padded, mul_routed_weight, top_k, block_m) -> ()  tg_fp8_moe_gemm
    fp8_quant_1x128(x) -> (q, scales)                                                   tg_fp8_quant_1x128
    fp8_fused_moe(hidden, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids) -> out   the FP8 MoE layer (tg_fp8_fused_moe
                                                                                        when it fits one chunk)
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

NAMESPACE = "tilegym_hip"
OP_NAMES = ("fp8_gemm", "fp8_gemm_out", "fp8_ragged_gemm", "fp8_moe_gemm_out", "fp8_quant_1x128", "fp8_fused_moe")


def _mnk(a: torch.Tensor, b: torch.Tensor, trans_a: bool, trans_b: bool) -> Tuple[int, int, int]:
    if a.dim() != 2 or b.dim() != 2:
        raise ValueError("fp8_gemm expects 2-D operands")
    M, K = (a.shape[1], a.shape[0]) if trans_a else (a.shape[0], a.shape[1])
    N, KB = (b.shape[0], b.shape[1]) if trans_b else (b.shape[1], b.shape[0])
    if K != KB:
        raise ValueError(f"Incompatible matrices: K dimension of A is {K}, K dimension of B is {KB}")
    return M, N, K


@torch.library.custom_op(f"{NAMESPACE}::fp8_gemm", mutates_args=(), device_types="cuda")
def fp8_gemm(a: torch.Tensor, b: torch.Tensor, scale_a: Optional[torch.Tensor], scale_b: Optional[torch.Tensor],
             trans_a: bool, trans_b: bool, alpha: float, out_dtype: torch.dtype) -> torch.Tensor:
    M, N, _ = _mnk(a, b, trans_a, trans_b)
    c = torch.empty((M, N), dtype=out_dtype, device=a.device)
    _lib.fp8_gemm(c, a, b, scale_a, scale_b, trans_a, trans_b, alpha, 0.0)
    return c


@fp8_gemm.register_fake
def _(a, b, scale_a, scale_b, trans_a, trans_b, alpha, out_dtype):
    M, N, _ = _mnk(a, b, trans_a, trans_b)
    return a.new_empty((M, N), dtype=out_dtype)


@torch.library.custom_op(f"{NAMESPACE}::fp8_gemm_out", mutates_args=("c",), device_types="cuda")
def fp8_gemm_out(c: torch.Tensor, a: torch.Tensor, b: torch.Tensor, scale_a: Optional[torch.Tensor],
                 scale_b: Optional[torch.Tensor], trans_a: bool, trans_b: bool, alpha: float, beta: float) -> None:
    _lib.fp8_gemm(c, a, b, scale_a, scale_b, trans_a, trans_b, alpha, beta)


@fp8_gemm_out.register_fake
def _(c, a, b, scale_a, scale_b, trans_a, trans_b, alpha, beta):
    M, N, _ = _mnk(a, b, trans_a, trans_b)
    if tuple(c.shape) != (M, N):
        raise ValueError(f"c must be ({M}, {N})")


@torch.library.custom_op(f"{NAMESPACE}::fp8_ragged_gemm", mutates_args=(), device_types="cuda")
def fp8_ragged_gemm(a: torch.Tensor, b: torch.Tensor, a_scale: Optional[torch.Tensor], b_scale: torch.Tensor,
                    m_indptr: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    # rows past m_indptr[-1] belong to no expert and are not written: they read as zero
    c = torch.zeros((a.shape[0], b.shape[1]), dtype=out_dtype, device=a.device)
    _lib.fp8_ragged_gemm(c, a, b, a_scale, b_scale, m_indptr)
    return c


@fp8_ragged_gemm.register_fake
def _(a, b, a_scale, b_scale, m_indptr, out_dtype):
    if a.dim() != 2 or b.dim() != 3 or a.shape[1] != b.shape[2]:
        raise ValueError("fp8_ragged_gemm expects a (rows, K) and b (experts, N, K)")
    return a.new_empty((a.shape[0], b.shape[1]), dtype=out_dtype)


@torch.library.custom_op(f"{NAMESPACE}::fp8_moe_gemm_out", mutates_args=("c",), device_types="cuda")
def fp8_moe_gemm_out(c: torch.Tensor, a: torch.Tensor, b: torch.Tensor, a_scale: Optional[torch.Tensor],
                     b_scale: Optional[torch.Tensor], topk_weights: Optional[torch.Tensor], sorted_token_ids: torch.Tensor,
                     expert_ids: torch.Tensor, num_tokens_post_padded: torch.Tensor, mul_routed_weight: bool, top_k: int,
                     block_m: int) -> None:
    _lib.fp8_moe_gemm(c.view(-1, c.shape[-1]), a, b, a_scale, b_scale, topk_weights, sorted_token_ids, expert_ids,
                      num_tokens_post_padded, mul_routed_weight, top_k, block_m)


@fp8_moe_gemm_out.register_fake
def _(c, a, b, a_scale, b_scale, topk_weights, sorted_token_ids, expert_ids, num_tokens_post_padded, mul_routed_weight,
      top_k, block_m):
    if b.dim() != 3 or a.shape[-1] != b.shape[2] or c.shape[-1] != b.shape[1]:
        raise ValueError("fp8_moe_gemm_out expects a (tokens, K), b (experts, N, K) and c (..., N)")


@torch.library.custom_op(f"{NAMESPACE}::fp8_quant_1x128", mutates_args=(), device_types="cuda")
def fp8_quant_1x128(x: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    q, scales = _lib.fp8_quant_1x128(x.contiguous(), 0.0, False)
    return q, scales


@fp8_quant_1x128.register_fake
def _(x):
    if x.shape[-1] % 128 != 0:
        raise ValueError("the last dimension must be a multiple of 128")
    return x.new_empty(x.shape, dtype=torch.float8_e4m3fn), x.new_empty(x.shape[:-1] + (x.shape[-1] // 128,), dtype=torch.float32)


@torch.library.custom_op(f"{NAMESPACE}::fp8_fused_moe", mutates_args=(), device_types="cuda")
def fp8_fused_moe(hidden: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w1_scale: torch.Tensor, w2_scale: torch.Tensor,
                  topk_weights: torch.Tensor, topk_ids: torch.Tensor) -> torch.Tensor:
    from .ops.moe_interface import fused_experts_impl
    return fused_experts_impl(hidden, w1, w2, topk_weights, topk_ids, inplace=False, use_fp8_w8a8=True, w1_scale=w1_scale,
                              w2_scale=w2_scale)


@fp8_fused_moe.register_fake
def _(hidden, w1, w2, w1_scale, w2_scale, topk_weights, topk_ids):
    if hidden.dim() != 2 or w1.dim() != 3 or w2.dim() != 3 or w1.shape[2] != hidden.shape[1] or w2.shape[1] != hidden.shape[1]:
        raise ValueError("fp8_fused_moe expects hidden (T, H), w1 (E, 2I, H) and w2 (E, H, I)")
    return hidden.new_empty(hidden.shape, dtype=torch.bfloat16 if hidden.dtype == torch.bfloat16 else torch.float16)


def registered_ops():
    """Names of the operators this module registered, as ``torch.ops`` sees them."""
    ns = getattr(torch.ops, NAMESPACE)
    return [f"{NAMESPACE}::{name}" for name in OP_NAMES if hasattr(ns, name)]
