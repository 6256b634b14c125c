"""The ``cl.*`` functions (``python/cleave/frontend/composites.py:10-63`` names and arguments).

Each works on two kinds of operand: on a traced ``cl.Tensor`` it records ops, on a torch tensor
it computes at once, so the body of a ``@jit`` function is also its own eager definition.  The
choice is made in one place (``_DUAL``: per function, the handle's method and torch's spelling);
what is built from other functions of this module (``rsqrt``, ``rms_norm``, ``softmax``) needs
no choice of its own.
"""

from __future__ import annotations

from typing import Optional

from .program import grouped_matmul
from .tensor import Tensor

# name -> (what to call on a traced handle, what to call on a torch tensor)
_DUAL = {
    "exp": (lambda x: x.exp(), lambda torch, x: torch.exp(x)),
    "sqrt": (lambda x: x.sqrt(), lambda torch, x: torch.sqrt(x)),
    "silu": (lambda x: x.silu(), lambda torch, x: torch.nn.functional.silu(x)),
    "max": (lambda x, dim, keepdim: x.max(dim, keepdim=keepdim),
            lambda torch, x, dim, keepdim: x.amax(dim, keepdim=keepdim)),       # values only, no indices
    "matmul": (lambda a, b: a @ b, lambda torch, a, b: grouped_matmul(a, b)),
}


def _dual(name, *operands):
    traced, eager = _DUAL[name]
    if any(isinstance(x, Tensor) for x in operands):
        return traced(*operands)
    import torch

    return eager(torch, *operands)


def exp(x):
    return _dual("exp", x)


def sqrt(x):
    return _dual("sqrt", x)


def silu(x):
    return _dual("silu", x)


def rsqrt(x):
    """Reciprocal square root, spelled with the two ops the vocabulary has."""
    return 1.0 / sqrt(x)


def matmul(a, b):
    """``a @ b``; leading (batch) extents may differ by a whole factor (grouped heads)."""
    return _dual("matmul", a, b)


def max(x, dim: int = -1, keepdim: bool = False):  # noqa: A001
    return _dual("max", x, dim, keepdim)


def sum(x, dim: int = -1, keepdim: bool = False):  # noqa: A001
    return x.sum(dim, keepdim=keepdim)          # both kinds of operand spell it alike


def mean(x, dim: int = -1, keepdim: bool = False):
    return x.mean(dim, keepdim=keepdim)


def rms_norm(x, dim: int = -1, eps: float = 0.0):
    """``x / sqrt(mean(x^2) [+ eps])`` along ``dim``; no learned weight."""
    power = mean(x * x, dim, keepdim=True)
    return x * rsqrt(power + eps if eps else power)


def softmax(x, dim: int = -1, shift: Optional[float] = None):
    """Without ``shift``: the exact form, ``exp(x - max x) / sum``.  With a number: ``exp(x +
    shift) / sum`` and no max op: mathematically the same function, but it can overflow."""
    if shift is None:
        x = x - max(x, dim, keepdim=True)
    elif shift:
        x = x + shift
    weights = exp(x)
    return weights / sum(weights, dim, keepdim=True)
