"""Built-in operators of ``autort.ops`` (filled in by the kernel modules)."""
from __future__ import annotations

from typing import Callable, Dict, Optional

_FACTORIES: Dict[str, Callable] = {}


def builtin(name: str):
    def deco(fn):
        _FACTORIES[name] = fn
        return fn
    return deco


def names():
    _load()
    return list(_FACTORIES)


def lookup(name: str):
    _load()
    f = _FACTORIES.get(name)
    return f() if f else None


_loaded = False


def _load():
    global _loaded
    if not _loaded:
        _loaded = True
        from . import builtin_ops  # noqa: F401  (registers the operators)
