"""Implementations registered under backend "hip" (one per public op)."""

from . import gemm, moe  # noqa: F401
