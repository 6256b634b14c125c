"""The vocabulary programs are written in: element types, named dimensions, argument
annotations, split requests, and the ``Tensor`` handle whose operators record ops.

The public names and spellings (``cl.f16``, ``cl.dims("M K")``, ``cl.Tensor["M", "K", cl.f16]``,
``cl.Scalar[cl.f32]``, ``cl.Split("K", (4, 8))``, ``batch + 1``, ``x.mT``, ``x | None``) are those
of ``python/cleave/frontend/tensor.py`` so that a program written for Cleave traces here as it
is.  A ``Tensor`` knows nothing about ops: every operator funnels into one call,
``owner.apply(kind, operands, **attributes)``, and the owner (a dense ``Program`` or a
``PagedProgram``) decides what that kind means for it.
"""

from __future__ import annotations

import numbers

from ..core.errors import SpecError


def is_number(x) -> bool:
    """A Python real that is not a bool."""
    return isinstance(x, numbers.Real) and not isinstance(x, bool)


def _is_count(x) -> bool:
    return isinstance(x, int) and not isinstance(x, bool)


# ================================================================================ element types
class DType:
    """An element type, named as torch names it."""

    __slots__ = ("name", "short", "itemsize")
    _by_spelling: dict = {}

    def __init__(self, name: str, short: str, itemsize: int):
        self.name, self.short, self.itemsize = name, short, itemsize
        for spelling in (name, short, "torch." + name):
            DType._by_spelling[spelling] = self

    @property
    def torch(self):
        import torch

        return getattr(torch, self.name)

    def __reduce__(self):                      # one object per type, also after a pickle round trip
        return (as_dtype, (self.name,))

    def __str__(self):
        return self.name

    def __repr__(self):
        return "cl." + self.short


f16 = DType("float16", "f16", 2)
bf16 = DType("bfloat16", "bf16", 2)
f32 = DType("float32", "f32", 4)
i32 = DType("int32", "i32", 4)


def as_dtype(value):
    """A ``DType`` for a ``DType``, a name (``"f16"``, ``"float16"``) or a ``torch.dtype``;
    ``None`` stays ``None``."""
    if value is None or isinstance(value, DType):
        return value
    found = DType._by_spelling.get(str(value))
    if found is None:
        raise SpecError(f"unsupported dtype {value!r}")
    return found


# ================================================================================ dimensions
class Dim:
    """A named extent.  ``size`` fixes it; a ``dynamic`` one is only known per call and is planned
    at ``hint``.  ``dim + k`` names the extent ``k`` larger (the length of a CSR row-pointer
    array over ``dim`` rows is ``dim + 1``)."""

    __slots__ = ("name", "size", "dynamic", "hint")

    def __init__(self, name: str, size=None, dynamic: bool = False, hint=None):
        object.__setattr__(self, "name", str(name))
        object.__setattr__(self, "size", None if size is None else int(size))
        object.__setattr__(self, "dynamic", bool(dynamic))
        object.__setattr__(self, "hint", None if hint is None else int(hint))

    def __setattr__(self, *_):
        raise AttributeError("cl.Dim is immutable; use .bind(size)")

    def _key(self):
        return (self.name, self.size, self.dynamic, self.hint)

    def __eq__(self, other):
        return isinstance(other, Dim) and self._key() == other._key()

    def __hash__(self):
        return hash(self._key())

    def __reduce__(self):
        return (Dim, self._key())

    @property
    def extent(self) -> int:
        """The size to plan with: the bound size, else the hint."""
        chosen = self.hint if self.size is None else self.size
        if chosen is None:
            raise SpecError(f"dim {self.name!r} has no size; bind it (shapes={{{self.name!r}: ...}})")
        return chosen

    @property
    def sized(self) -> bool:
        return self.size is not None or self.hint is not None

    def bind(self, size) -> "Dim":
        return Dim(self.name, size, self.dynamic, self.hint)

    def __add__(self, k):
        if not _is_count(k):
            return NotImplemented
        grown = [n if n is None else n + k for n in (self.size, self.hint)]
        return Dim(f"{self.name}{k:+d}", grown[0], self.dynamic, grown[1])

    __radd__ = __add__

    def __repr__(self):
        shown = [repr(self.name)]
        shown += [f"{field}={getattr(self, field)!r}" for field in ("size", "hint") if getattr(self, field) is not None]
        if self.dynamic:
            shown.append("dynamic=True")
        return "Dim(" + ", ".join(shown) + ")"


def dims(names: str, dynamic: bool = False) -> tuple:
    """``M, K = cl.dims("M K")`` (commas work too)."""
    return tuple(Dim(word, dynamic=dynamic) for word in names.replace(",", " ").split())


def extent(d) -> int:
    """Planning size of a ``Dim`` or a literal extent."""
    return d.extent if isinstance(d, Dim) else int(d)


def dim_name(d):
    """The name of a ``Dim``; ``None`` for a literal extent."""
    return d.name if isinstance(d, Dim) else None


# ================================================================================ annotations
class TensorSpec:
    """What ``cl.Tensor[...]`` evaluates to; ``spec | None`` marks the argument optional."""

    __slots__ = ("dims", "dtype", "optional")

    def __init__(self, dims, dtype=None, optional: bool = False):
        self.dims, self.dtype, self.optional = tuple(dims), dtype, bool(optional)

    def __or__(self, other):
        return TensorSpec(self.dims, self.dtype, True) if other is None else NotImplemented

    __ror__ = __or__

    def __eq__(self, other):
        return isinstance(other, TensorSpec) and \
            (self.dims, self.dtype, self.optional) == (other.dims, other.dtype, other.optional)

    def __hash__(self):
        return hash((self.dims, self.dtype, self.optional))

    def __repr__(self):
        inner = ", ".join([dim_name(d) or str(d) for d in self.dims] + ([repr(self.dtype)] if self.dtype else []))
        return f"cl.Tensor[{inner}]" + (" | None" if self.optional else "")


class ScalarSpec:
    """What ``cl.Scalar[...]`` evaluates to."""

    __slots__ = ("dtype",)
    optional = False

    def __init__(self, dtype):
        self.dtype = dtype

    def __eq__(self, other):
        return isinstance(other, ScalarSpec) and self.dtype == other.dtype

    def __hash__(self):
        return hash(("scalar", self.dtype))

    def __repr__(self):
        return f"cl.Scalar[{self.dtype!r}]"


class Scalar:
    """``cl.Scalar[cl.f32]``: a number handed over at call time (paged programs)."""

    def __class_getitem__(cls, dtype):
        return ScalarSpec(as_dtype(dtype))


# ================================================================================ split requests
class Split:
    """A dimension the search may cut (split-K, split-KV) and the factors it should try."""

    __slots__ = ("dim", "factors")

    def __init__(self, dim, factors=(4, 8, 16)):
        object.__setattr__(self, "dim", dim_name(dim) or str(dim))
        object.__setattr__(self, "factors", tuple(int(f) for f in factors))

    def __setattr__(self, *_):
        raise AttributeError("cl.Split is immutable")

    def __eq__(self, other):
        return isinstance(other, Split) and (self.dim, self.factors) == (other.dim, other.factors)

    def __hash__(self):
        return hash((self.dim, self.factors))

    def __reduce__(self):
        return (Split, (self.dim, self.factors))

    def __repr__(self):
        return f"Split({self.dim!r}, {self.factors!r})"


def _each_split(request):
    """A split request is nothing, one item (a name, a ``Dim``, a ``Split``) or several."""
    if request is None or request is False:
        return ()
    return (request,) if isinstance(request, (str, Dim, Split)) else tuple(request)


def as_splits(request) -> tuple:
    """The request as ``Split`` objects (default factors where only a dimension was named)."""
    return tuple(item if isinstance(item, Split) else Split(item) for item in _each_split(request))


def split_names(request) -> tuple:
    """The dimension names of a request, each once, in the order given."""
    return tuple(dict.fromkeys(Split(item).dim if not isinstance(item, Split) else item.dim
                               for item in _each_split(request)))


# ================================================================================ the handle
class Tensor:
    """One value of a program under construction (and, subscripted, an argument annotation).

    ``program``: the owner; ``id``: the value's number there; ``dims``: ``Dim`` objects and
    literal extents.  ``_trans`` marks the ``.mT`` view, which exists only to be a matmul operand.
    """

    __array_priority__ = 1000        # numpy scalars defer to these operators

    def __class_getitem__(cls, items):
        shape, dtype = [], None
        for item in (items if isinstance(items, tuple) else (items,)):
            if isinstance(item, DType):
                dtype = item
            elif isinstance(item, str):
                shape.append(Dim(item))
            elif isinstance(item, Dim) or _is_count(item):
                shape.append(item)
            else:
                raise TypeError(f"bad cl.Tensor annotation item {item!r}")
        return TensorSpec(shape, dtype)

    def __init__(self, program, id: int, dims, dtype: DType, trans: bool = False):  # noqa: A002
        self.program, self.id, self.dims, self.dtype, self._trans = program, id, tuple(dims), dtype, trans

    shape = property(lambda self: tuple(extent(d) for d in self.dims))
    ndim = property(lambda self: len(self.dims))

    def __repr__(self):
        axes = ", ".join(dim_name(d) or str(d) for d in self.dims)
        return f"Tensor(%{self.id}{'.mT' if self._trans else ''}[{axes}] {self.dtype!r})"

    def __bool__(self):
        raise SpecError("data-dependent control flow on a traced cl.Tensor")

    # ---- views
    @property
    def mT(self) -> "Tensor":  # noqa: N802
        if self.ndim < 2:
            raise SpecError(".mT needs a tensor of rank >= 2")
        *lead, rows, cols = self.dims
        return Tensor(self.program, self.id, (*lead, cols, rows), self.dtype, not self._trans)

    @property
    def T(self) -> "Tensor":  # noqa: N802
        if self.ndim != 2:
            raise SpecError(".T is only defined for 2-D tensors; use .mT")
        return self.mT

    def view(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        return self.program.apply("view", (self,), shape=tuple(shape))

    # ---- ops with their own argument conventions
    def __matmul__(self, other):
        return self.program.apply("matmul", (self, other))

    def __rmatmul__(self, other):
        return self.program.apply("matmul", (other, self))

    def __neg__(self):
        return self * -1.0

    def __sub__(self, other):                 # x - 3 is recorded as x + (-3)
        return self + (-float(other)) if is_number(other) else self.program.apply("sub", (self, other))

    def __rsub__(self, other):
        return -self + float(other) if is_number(other) else self.program.apply("sub", (other, self))

    def __pow__(self, power):
        rewritten = {2: lambda: self * self, 0.5: self.sqrt, -0.5: self.rsqrt}.get(power)
        if rewritten is None:
            raise SpecError(f"x ** {power!r}: only 2, 0.5 and -0.5 are lowerable")
        return rewritten()

    def rsqrt(self):
        return 1.0 / self.sqrt()

    def _reduce(self, kind, dim, keepdim):
        if not keepdim:
            raise SpecError("tile-IR reductions keep the reduced axis; pass keepdim=True")
        return self.program.apply(kind, (self,), dim=dim)

    def sum(self, dim: int = -1, keepdim: bool = False):
        return self._reduce("reduce_sum", dim, keepdim)

    def max(self, dim: int = -1, keepdim: bool = False):
        return self._reduce("reduce_max", dim, keepdim)

    def mean(self, dim: int = -1, keepdim: bool = False):
        return self.sum(dim, keepdim) / float(self.shape[dim])


def _install_operators():
    """The uniform operators: ``x + y`` / ``y + x`` -> ``apply("add", ...)`` and so on."""
    def binary(kind, swapped):
        def method(self, other):
            return self.program.apply(kind, (other, self) if swapped else (self, other))
        return method

    for kind, forward, reflected in (("add", "__add__", "__radd__"), ("mul", "__mul__", "__rmul__"),
                                     ("div", "__truediv__", "__rtruediv__")):
        setattr(Tensor, forward, binary(kind, False))
        setattr(Tensor, reflected, binary(kind, True))
    for kind in ("exp", "sqrt", "silu"):
        setattr(Tensor, kind, (lambda k: lambda self: self.program.apply(k, (self,)))(kind))


_install_operators()
