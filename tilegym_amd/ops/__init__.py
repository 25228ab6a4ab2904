"""tilegym.ops-shaped namespace: public stubs + the "hip" implementations (registered on import)."""

from . import hip  # noqa: F401  (registers implementations)
from .moe_interface import fused_experts_impl, fused_moe, invoke_fused_moe_kernel, moe_align_block_size
from .ops import group_gemm, matmul

__all__ = ["matmul", "group_gemm", "fused_moe", "fused_experts_impl", "invoke_fused_moe_kernel", "moe_align_block_size"]
