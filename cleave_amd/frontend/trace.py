"""``trace(fn, shapes, dtype)``: call an annotated function on proxies and return the
``Program`` it recorded (``python/cleave/frontend/trace.py:23-74``)."""

from __future__ import annotations

import inspect

from ..core.errors import SpecError
from .program import Program
from .tensor import Dim, ScalarSpec, Tensor, TensorSpec, as_dtype, as_splits, f16


def _parameters(fn):
    return list(inspect.signature(fn, eval_str=True).parameters.values())


def signature_dims(fn) -> dict:
    """Named dims of ``fn``'s ``cl.Tensor[...]`` annotations, in order of first appearance."""
    found = {}
    for p in _parameters(fn):
        if isinstance(p.annotation, TensorSpec):
            for d in p.annotation.dims:
                if isinstance(d, Dim) and d.name not in found:
                    found[d.name] = d
    return found


def _as_outputs(result, fn_name):
    if isinstance(result, dict):
        pairs = list(result.items())
    elif isinstance(result, (tuple, list)):
        pairs = [(None, r) for r in result]
    else:
        pairs = [(None, result)]
    for _, r in pairs:
        if not isinstance(r, Tensor):
            raise SpecError(f"{fn_name} must return cl.Tensor(s), got {type(r).__name__}")
    return pairs


def trace(fn, shapes: dict | None = None, dtype=None, *, split=None, name=None):
    """A ``Program``; for a function with ``cl.Scalar`` / optional tensor arguments, a
    ``PagedProgram`` (whose dims are all dynamic, so ``shapes`` must be empty)."""
    from .jit import JitFunction
    from .paged import is_paged, trace_paged

    if is_paged(fn):
        if shapes:
            raise SpecError(f"{getattr(fn, '__name__', fn)}: paged dims are dynamic; drop shapes=")
        return trace_paged(fn, dtype, name=name, split=split)
    if isinstance(fn, JitFunction):
        dtype = dtype or fn.dtype
        split = fn.split if split is None else split
        name = name or fn.__name__
        fn = fn.fn
    shapes = dict(shapes or {})
    declared = signature_dims(fn)
    stray = sorted(set(shapes) - set(declared))
    if stray:
        raise SpecError(f"{fn.__name__}: shapes {stray} are not dims of the signature (dims: {list(declared)})")
    program = Program(name or fn.__name__, as_dtype(dtype) or f16)
    program.split = as_splits(split)
    call_args = []
    for p in _parameters(fn):
        note = p.annotation
        if isinstance(note, TensorSpec):
            bound = []
            for d in note.dims:
                if isinstance(d, Dim):
                    if d.name in shapes:
                        d = d.bind(shapes[d.name])
                    if d.size is None and d.hint is None:
                        raise SpecError(f"{fn.__name__}: dim {d.name!r} of {p.name!r} unbound; "
                                        f"pass shapes={{{d.name!r}: ...}}")
                bound.append(d)
            call_args.append(program.input(p.name, bound, note.dtype))
        elif isinstance(note, ScalarSpec):
            raise NotImplementedError(f"{p.name}: runtime cl.Scalar arguments are not in the tile IR yet")
        elif p.default is not inspect.Parameter.empty:
            call_args.append(p.default)
        else:
            raise SpecError(f"{fn.__name__}: annotate {p.name!r} with cl.Tensor[...] or give it a default")
    for out_name, t in _as_outputs(fn(*call_args), fn.__name__):
        program.output(t, out_name)
    return program
