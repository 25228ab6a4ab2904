""" "hip" implementations of the MoE entry points."""

from __future__ import annotations

import torch

from ... import _lib
from ...backend import register_impl

FP8 = torch.float8_e4m3fn


@register_impl("invoke_fused_moe_kernel", backend="hip")
def invoke_fused_moe_kernel(A, B, C, A_scale, B_scale, topk_weights, topk_ids, sorted_token_ids,
                            expert_ids, num_tokens_post_padded, mul_routed_weight, top_k, config,
                            compute_type=None, use_fp8_w8a8=True, use_int8_w8a16=False,
                            block_shape=None, **kwargs) -> None:
    """Token-gather block-scaled FP8 GEMM (src/tilegym/ops/tilecpp/moe.py:241-310): row r of the
    sorted slot list reads A[id // top_k], multiplies with B[expert_ids[r // BLOCK_SIZE_M]] and
    writes C[id] (id = sorted_token_ids[r]); padding slots (id >= numel(topk_ids)) are skipped."""
    if use_int8_w8a16:
        raise NotImplementedError("int8 weights are not implemented by the hip backend")
    if not use_fp8_w8a8 or A.dtype != FP8 or B.dtype != FP8:
        raise NotImplementedError("the hip backend implements the use_fp8_w8a8 path only "
                                  "(float8_e4m3fn activations and weights)")
    if block_shape is not None and tuple(block_shape) != (128, 128):
        raise NotImplementedError("the hip backend implements 128x128 quantization blocks only")
    assert topk_weights is None or topk_weights.stride(1) == 1
    assert sorted_token_ids.stride(0) == 1
    assert A.is_contiguous() and B.is_contiguous() and C.is_contiguous()
    block_m = int(config.get("BLOCK_SIZE_M", config.get("TILE_SIZE_M", 128)))
    num_valid = topk_ids.numel()
    N = B.shape[1]
    c2 = C.view(-1, N)
    assert c2.shape[0] == num_valid, "C must provide one row per (token, k) slot"
    w = None
    if mul_routed_weight:
        w = topk_weights.reshape(-1).float().contiguous()
    a_s = None if A_scale is None else A_scale.float().contiguous()
    b_s = None if B_scale is None else B_scale.float().contiguous()
    _lib.fp8_moe_gemm(c2, A, B, a_s, b_s, w, sorted_token_ids.to(torch.int32),
                      expert_ids.to(torch.int32), num_tokens_post_padded.reshape(-1).to(torch.int32),
                      bool(mul_routed_weight), int(top_k), block_m, kwargs.get("kernel_configs"))
    return None


@register_impl("moe_align_block_size", backend="hip")
def moe_align_block_size(topk_ids: torch.Tensor, block_size: int, num_experts: int):
    """Device-side token alignment, no host synchronisation; same outputs and buffer sizes as
    src/tilegym/ops/cutile/moe_align_block.py:205-268: (sorted_ids[numel + E*(bs-1)] pre-filled
    with the sentinel numel, expert_ids[ceil(that/bs)], num_tokens_post_pad[1], cumsum[E+1] of
    padded counts, max_expert_cnt[1]).  Stable within an expert.  One HIP launch for up to 512
    experts; more raise NotImplementedError."""
    if not topk_ids.is_cuda:
        raise RuntimeError("the hip backend works on device tensors only; topk_ids is on " + str(topk_ids.device))
    if num_experts > _lib.MOE_ALIGN_MAX_EXPERTS:
        raise NotImplementedError(f"moe_align_block_size on the hip backend handles up to {_lib.MOE_ALIGN_MAX_EXPERTS} experts "
                                  f"(one launch, per-expert counters in LDS); got {num_experts}")
    if topk_ids.numel() == 0:  # nothing routed: every output is its fill value (no kernel needed)
        dev = topk_ids.device
        cap = num_experts * (block_size - 1)
        nblk = -(-cap // block_size)
        return (torch.zeros(cap, dtype=torch.int32, device=dev), torch.zeros(nblk, dtype=torch.int32, device=dev),
                torch.zeros(1, dtype=torch.int32, device=dev), torch.zeros(num_experts + 1, dtype=torch.int32, device=dev),
                torch.zeros(1, dtype=torch.int32, device=dev))
    return _lib.moe_align_block_size(topk_ids, block_size, num_experts)
