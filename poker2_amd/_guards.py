"""Argument guards that stay in force under ``python -O``.

The kernels index device memory with the sizes and row numbers their callers pass; a wrong
shape, dtype or row bound must stop on the host, not as a memory fault on the GPU.  A plain
``assert`` is compiled out by ``-O``, so the wrappers call ``require`` instead.  It raises
``AssertionError``, which is what the reference's wrappers raise for the same mistakes.
"""
from __future__ import annotations


def require(condition, what: str) -> None:
    if not condition:
        raise AssertionError(what)
