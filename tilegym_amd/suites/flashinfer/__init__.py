"""FlashInfer-suite FP8 GEMM ops (as in src/tilegym/suites/flashinfer/__init__.py:31-32)."""

from . import ops  # noqa: F401

__all__ = ["ops"]
