"""``trace(fn, shapes, dtype)``: run an annotated function on handles and keep what it recorded
(the call of ``python/cleave/frontend/trace.py:23-74``).

A function whose signature has a ``cl.Scalar`` or an optional tensor is a paged operator: all
its dimensions are dynamic, so it takes no ``shapes`` and is handed to ``paged.trace_paged``.
"""

from __future__ import annotations

import inspect
from typing import Optional

from ..core.errors import SpecError
from .program import Program
from .tensor import Dim, ScalarSpec, Tensor, TensorSpec, as_dtype, as_splits, f16


def annotated_parameters(fn) -> list:
    """``inspect`` parameters with string annotations evaluated."""
    return list(inspect.signature(fn, eval_str=True).parameters.values())


def signature_dims(fn) -> dict:
    """name -> ``Dim`` for every named dimension in ``fn``'s tensor annotations, first mention first."""
    found = {}
    for parameter in annotated_parameters(fn):
        if isinstance(parameter.annotation, TensorSpec):
            for d in parameter.annotation.dims:
                if isinstance(d, Dim):
                    found.setdefault(d.name, d)
    return found


def named_results(result, fn_name: str) -> list:
    """What a traced body returned, as ``(name | None, handle)`` pairs: a dict names its outputs,
    a tuple / list / single handle leaves the naming to the program."""
    if isinstance(result, dict):
        pairs = list(result.items())
    else:
        pairs = [(None, r) for r in (result if isinstance(result, (tuple, list)) else [result])]
    for _, handle in pairs:
        if not isinstance(handle, Tensor):
            raise SpecError(f"{fn_name} must return cl.Tensor(s), got {type(handle).__name__}")
    return pairs


def unwrap(fn, dtype=None, split=None, name=None):
    """``(plain function, dtype, split, name)`` with a ``JitFunction``'s own settings filled in
    where the caller gave none."""
    from .jit import JitFunction

    if isinstance(fn, JitFunction):
        dtype, name = dtype or fn.dtype, name or fn.__name__
        split = fn.split if split is None else split
        fn = fn.fn
    return fn, dtype, split, name or fn.__name__


def trace(fn, shapes: Optional[dict] = None, dtype=None, *, split=None, name=None):
    from .paged import is_paged, trace_paged

    if is_paged(fn):
        if shapes:
            raise SpecError(f"{getattr(fn, '__name__', fn)}: paged dims are dynamic; drop shapes=")
        return trace_paged(fn, dtype, name=name, split=split)
    fn, dtype, split, name = unwrap(fn, dtype, split, name)
    sizes = dict(shapes or {})
    unknown = sorted(set(sizes) - set(signature_dims(fn)))
    if unknown:
        raise SpecError(f"{fn.__name__}: shapes {unknown} are not dims of the signature "
                        f"(dims: {list(signature_dims(fn))})")
    program = Program(name, as_dtype(dtype) or f16)
    program.split = as_splits(split)

    def sized(d, owner):
        if not isinstance(d, Dim):
            return d
        d = d.bind(sizes[d.name]) if d.name in sizes else d
        if not d.sized:
            raise SpecError(f"{fn.__name__}: dim {d.name!r} of {owner!r} unbound; pass shapes={{{d.name!r}: ...}}")
        return d

    handles = []
    for parameter in annotated_parameters(fn):
        note = parameter.annotation
        if isinstance(note, TensorSpec):
            handles.append(program.input(parameter.name, [sized(d, parameter.name) for d in note.dims], note.dtype))
        elif isinstance(note, ScalarSpec):
            raise NotImplementedError(f"{parameter.name}: runtime cl.Scalar arguments are not in the tile IR yet")
        elif parameter.default is not inspect.Parameter.empty:
            handles.append(parameter.default)
        else:
            raise SpecError(f"{fn.__name__}: annotate {parameter.name!r} with cl.Tensor[...] or give it a default")
    for out_name, handle in named_results(fn(*handles), fn.__name__):
        program.output(handle, out_name)
    return program
