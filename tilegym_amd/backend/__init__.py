"""Backend registry and dispatcher with the semantics of the reference's plugin boundary
(src/tilegym/backend/dispatcher.py:34-141, src/tilegym/backend/selector.py:185-215), reduced
to the single backend this package ships: ``"hip"``.

An implementation registers itself with ``@register_impl(name, backend)``; a public op is a
stub decorated with ``@dispatch(name)`` whose wrapper pops an optional ``backend=`` keyword,
looks the implementation up by (name, backend) and calls it with the caller's arguments
untouched.  There is no fallback backend here: a missing implementation raises
``NotImplementedError`` (the reference's behaviour under ``DISABLE_FALLBACK=1``).
"""

from __future__ import annotations

import functools
import logging
import os
from typing import Callable, Dict, List

logger = logging.getLogger("tilegym_amd.backend")

BACKEND_ENV = "CUTILE_TUTORIALS_BACKEND"  # same variable the reference reads (selector.py:208-215)
_KNOWN_BACKENDS = ("hip",)
_DEFAULT_BACKEND = "hip"

_REGISTRY: Dict[str, Dict[str, Callable]] = {}
_current_backend = None


def _hip_library_present() -> bool:
    from .. import _lib

    return _lib.is_built()


def is_backend_available(backend: str) -> bool:
    """True when ``backend`` can run here: only "hip", and only once its library is built."""
    return backend == "hip" and _hip_library_present()


def get_available_backends() -> List[str]:
    return [b for b in _KNOWN_BACKENDS if is_backend_available(b)]


def set_backend(backend: str) -> None:
    """Select the global backend; raises ValueError for an unknown or unavailable one
    (src/tilegym/backend/selector.py:212-215)."""
    global _current_backend
    if backend not in _KNOWN_BACKENDS:
        raise ValueError(f"Unknown backend '{backend}'. Available backends: {list(_KNOWN_BACKENDS)}")
    if not is_backend_available(backend):
        raise ValueError(f"Backend '{backend}' is not available: libtilegym_hip.so has not been built")
    _current_backend = backend


def get_current_backend() -> str:
    global _current_backend
    if _current_backend is None:
        requested = os.environ.get(BACKEND_ENV)
        if requested is not None and requested not in _KNOWN_BACKENDS:
            raise ValueError(f"{BACKEND_ENV}={requested!r}: this build only provides {list(_KNOWN_BACKENDS)}")
        _current_backend = requested or _DEFAULT_BACKEND
    return _current_backend


def register_impl(name: str, backend: str):
    """Register ``func`` as the ``backend`` implementation of op ``name``."""

    def decorator(func):
        _REGISTRY.setdefault(name, {})[backend] = func
        logger.debug("registered '%s' implementation for '%s'", backend, name)
        return func

    return decorator


def dispatch(name: str, fallback_backend: str = None):
    """Turn a stub into a dispatcher for op ``name``."""

    def decorator(default_impl):
        @functools.wraps(default_impl)
        def wrapper(*args, **kwargs):
            explicit = kwargs.pop("backend", None)
            backend = explicit if explicit is not None else get_current_backend()
            impls = _REGISTRY.get(name, {})
            if backend in impls:
                logger.debug("dispatch '%s' -> '%s'", name, backend)
                return impls[backend](*args, **kwargs)
            raise NotImplementedError(
                f"No implementation of '{name}' for backend '{backend}' "
                f"(registered: {sorted(k for k in impls if k != 'default')})")

        _REGISTRY.setdefault(name, {})["default"] = default_impl
        wrapper._tilegym_op_name = name
        return wrapper

    return decorator


def get_available_backends_for_op(name: str) -> list:
    return sorted(k for k in _REGISTRY.get(name, {}) if k != "default")


def get_registry_info() -> Dict[str, List[str]]:
    return {name: sorted(impls) for name, impls in _REGISTRY.items()}


__all__ = [
    "dispatch", "register_impl", "set_backend", "get_current_backend", "is_backend_available",
    "get_available_backends", "get_available_backends_for_op", "get_registry_info",
]
