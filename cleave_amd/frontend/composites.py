"""The ``cl.*`` functions.  Given traced ``cl.Tensor`` handles they record ops; given torch
tensors they compute eagerly, so the body of a ``@cleave.jit`` function doubles as its own
eager definition (``python/cleave/frontend/composites.py:10-63``)."""

from __future__ import annotations

from .program import grouped_matmul
from .tensor import Tensor


def _torch():
    import torch

    return torch


def _is_traced(*xs) -> bool:
    return any(isinstance(x, Tensor) for x in xs)


def exp(x):
    return x.exp() if _is_traced(x) else _torch().exp(x)


def sqrt(x):
    return x.sqrt() if _is_traced(x) else _torch().sqrt(x)


def silu(x):
    return x.silu() if _is_traced(x) else _torch().nn.functional.silu(x)


def rsqrt(x):
    """``1 / sqrt(x)``; the op vocabulary has no rsqrt of its own."""
    return 1.0 / sqrt(x)


def matmul(a, b):
    """``a @ b`` with grouped broadcast of the leading (batch) dims."""
    return a @ b if _is_traced(a, b) else grouped_matmul(a, b)


def sum(x, dim: int = -1, keepdim: bool = False):  # noqa: A001
    return x.sum(dim, keepdim=keepdim)


def max(x, dim: int = -1, keepdim: bool = False):  # noqa: A001
    """Values of the max over ``dim`` (no indices)."""
    if _is_traced(x):
        return x.max(dim, keepdim=keepdim)
    return x.amax(dim, keepdim=keepdim)


def mean(x, dim: int = -1, keepdim: bool = False):
    return x.mean(dim, keepdim=keepdim)


def rms_norm(x, dim: int = -1, eps: float = 0.0):
    """``x * rsqrt(mean(x * x) + eps)``, no learned weight."""
    ms = mean(x * x, dim, keepdim=True)
    if eps:
        ms = ms + eps
    return x * rsqrt(ms)


def softmax(x, dim: int = -1, shift: float | None = None):
    """``shift=None``: exact ``exp(x - max x) / sum``.  A number: ``exp(x + shift) / sum`` with
    no max op (the same function mathematically; it overflows where the exact form cannot)."""
    if shift is None:
        e = exp(x - max(x, dim, keepdim=True))
    elif shift:
        e = exp(x + shift)
    else:
        e = exp(x)
    return e / sum(e, dim, keepdim=True)
