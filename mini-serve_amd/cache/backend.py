"""Choice of the page bookkeeping implementation: ``python`` (default) or ``cpp`` (the C++ block
core built from ``csrc/block_core.cpp``), by argument or the environment variable
``MINISERVE_BLOCK_BACKEND`` as in the reference (miniserve/cache/backend.py:46-94)."""

from __future__ import annotations

import os

BACKENDS = ("python", "cpp")
ENV = "MINISERVE_BLOCK_BACKEND"


def backend_name(name: str | None = None) -> str:
    name = name or os.environ.get(ENV) or "python"
    if name not in BACKENDS:
        raise ValueError(f"unknown block backend {name!r}, expected one of {BACKENDS}")
    return name


def allocator_class(name: str | None = None):
    if backend_name(name) == "cpp":
        from .native import NativePageAllocator

        return NativePageAllocator
    from .pages import PageAllocator

    return PageAllocator
