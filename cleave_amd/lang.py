"""The program-writing vocabulary, meant to be imported as ``import cleave_amd.lang as cl``.

It gathers, under the short names programs are written with (those of ``python/cleave/lang.py``):
element types and dimensions, argument annotations, the op functions, the paged-attention
declarations, plus two names that are looked up late because their homes import torch
(``Tolerance``) or the operator registry (``workloads``).
"""

import importlib

from .frontend import composites as _ops
from .frontend import paged as _paged
from .frontend import tensor as _tensor

_EAGER = {
    _tensor: "DType Dim Scalar Split Tensor bf16 dims f16 f32 i32",
    _ops: "exp matmul max mean rms_norm rsqrt silu sqrt sum",
    _paged: "PageTable ScheduleHints paged_gather softmax",
}
_LATE = {"Tolerance": (".runtime.validate", "Tolerance"), "workloads": (".frontend.paged", "workloads")}

for _module, _names in _EAGER.items():
    for _name in _names.split():
        globals()[_name] = getattr(_module, _name)

__all__ = sorted([name for names in _EAGER.values() for name in names.split()] + list(_LATE))


def __getattr__(name):
    if name not in _LATE:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    module, attribute = _LATE[name]
    return getattr(importlib.import_module(module, __package__), attribute)
