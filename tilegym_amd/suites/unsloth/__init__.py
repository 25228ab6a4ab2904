"""Unsloth-suite FP8 ops (re-exported as in src/tilegym/suites/unsloth/__init__.py:32)."""

from . import ops  # noqa: F401
from .ops import act_quant, w8a8_block_fp8_matmul, weight_dequant

__all__ = ["ops", "act_quant", "weight_dequant", "w8a8_block_fp8_matmul"]
