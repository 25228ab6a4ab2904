"""tilegym_amd -- MI355X (gfx950) FP8 GEMM behind the TileGym op API.

Import paths mirror the reference package (src/tilegym/__init__.py:34-49):
``tilegym_amd.ops.matmul``, ``tilegym_amd.ops.group_gemm``,
``tilegym_amd.ops.moe_interface.invoke_fused_moe_kernel``,
``tilegym_amd.suites.unsloth.ops.w8a8_block_fp8_matmul``,
``tilegym_amd.suites.flashinfer.ops.{ragged_block_scaled_bmm,gemm_alpha_beta}``,
``tilegym_amd.set_backend`` / ``is_backend_available``.  ``install_as_tilegym()`` makes the same
modules importable under the name ``tilegym``.  Importing the package also registers the GEMM entry points with
torch's dispatcher as ``torch.ops.tilegym_hip.*`` (``tilegym_amd.torch_ops``).
"""

from __future__ import annotations

import sys

__version__ = "0.1.0"

from .backend import (dispatch, get_available_backends, get_current_backend,  # noqa: F401
                      get_registry_info, is_backend_available, register_impl, set_backend)
from . import ops, suites  # noqa: F401,E402
from . import torch_ops  # noqa: F401,E402  (registers torch.ops.tilegym_hip.*)


def install_as_tilegym() -> None:
    """Alias this package as ``tilegym`` in ``sys.modules`` so that code written against the
    reference's import paths (``from tilegym.suites import unsloth`` ...) runs unchanged.
    Refuses to shadow a real ``tilegym`` that is already imported."""
    existing = sys.modules.get("tilegym")
    this = sys.modules[__name__]
    if existing is not None and existing is not this:
        raise RuntimeError("a different 'tilegym' package is already imported")
    prefix = __name__ + "."
    for name, mod in list(sys.modules.items()):
        if name == __name__:
            sys.modules["tilegym"] = mod
        elif name.startswith(prefix):
            sys.modules["tilegym." + name[len(prefix):]] = mod


__all__ = ["ops", "suites", "dispatch", "register_impl", "set_backend", "get_current_backend",
           "is_backend_available", "get_available_backends", "get_registry_info", "install_as_tilegym"]
