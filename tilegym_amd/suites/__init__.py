"""tilegym.suites-shaped namespace (unsloth and flashinfer FP8 GEMM ops)."""

from . import flashinfer, unsloth  # noqa: F401
