"""Public op stubs with the reference's signatures (src/tilegym/ops/ops.py:715-773).
Bodies only raise; the registered "hip" implementation does the work."""

from __future__ import annotations

from typing import Any, List, Optional

import torch

from ..backend import dispatch, get_current_backend


@dispatch("matmul")
def matmul(
    a: torch.Tensor,
    b: torch.Tensor,
    trans_a: Optional[bool] = None,
    trans_b: Optional[bool] = None,
    static_persistent: Optional[bool] = True,
    use_tma: Optional[bool] = None,
    **kwargs: Any,
):
    """Matrix multiplication (src/tilegym/ops/ops.py:715-741).

    a: (M,K), or (K,M) with trans_a;  b: (K,N), or (N,K) with trans_b.  Without extra keywords
    the result has ``a.dtype``, as in the reference (src/tilegym/ops/cutile/matmul.py:446).
    Keyword-only extensions of the "hip" backend for scaled FP8:
      scale_a, scale_b : float | 1-element fp32 tensor (per-tensor) | block scales
                         (M, ceil(K/128)) and (ceil(N/128), ceil(K/128))
      out_dtype        : torch.bfloat16 / float16 / float32
      kernel_configs   : dict of schedule overrides (KERNEL, BLOCK_M, BLOCK_N, SPLIT_K, ROW_GROUPS)
    ``static_persistent`` and ``use_tma`` are accepted and ignored (no such choice on gfx950)."""
    raise NotImplementedError(f"Matmul is not implemented for this backend: {get_current_backend()}")


@dispatch("group_gemm")
def group_gemm(
    group_A: List[torch.Tensor],
    group_B: List[torch.Tensor],
    static_persistent: Optional[bool] = True,
    use_tma: Optional[bool] = True,
    **kwargs: Any,
):
    """List of independent GEMMs (src/tilegym/ops/ops.py:744-773); ``transpose_b`` keyword as in
    src/tilegym/ops/cutile/group_gemm.py:170-197.  "hip" extensions: ``scales_a``/``scales_b``
    (lists, per-tensor or block), ``out_dtype``, ``kernel_configs``."""
    raise NotImplementedError(f"Group GEMM is not implemented for this backend: {get_current_backend()}")
