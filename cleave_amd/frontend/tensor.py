"""Symbolic tensors, dims, dtypes and annotations of the ``cleave.lang`` surface.

Same public names and call signatures as the reference's
``python/cleave/frontend/tensor.py`` (``DType``, ``Dim``, ``dims``, ``Tensor[...]``
annotations, ``Scalar[...]``, ``Split``), so a ``@cleave.jit`` function written against
``import cleave.lang as cl`` traces unchanged.  A ``Tensor`` is only a handle: every
operator is forwarded to the builder (a ``Program`` or ``PagedProgram``) that owns it.
"""

from __future__ import annotations

import dataclasses
import numbers

from ..core.errors import SpecError


# ----------------------------------------------------------------------------- dtypes
@dataclasses.dataclass(frozen=True)
class DType:
    name: str  # torch's spelling: float16, bfloat16, float32, int32

    @property
    def short(self) -> str:
        return _ABBREV.get(self.name, self.name)

    @property
    def torch(self):
        import torch

        return getattr(torch, self.name)

    @property
    def itemsize(self) -> int:
        return {"float16": 2, "bfloat16": 2, "float32": 4, "int32": 4}[self.name]

    def __repr__(self):
        return f"cl.{self.short}"

    def __str__(self):
        return self.name


_ABBREV = {"float16": "f16", "bfloat16": "bf16", "float32": "f32", "int32": "i32"}
f16 = DType("float16")
bf16 = DType("bfloat16")
f32 = DType("float32")
i32 = DType("int32")
_LOOKUP = {}
for _d in (f16, bf16, f32, i32):
    _LOOKUP[_d.name] = _d
    _LOOKUP[_d.short] = _d


def as_dtype(value):
    """``None`` and ``DType`` pass through; strings and ``torch.dtype`` objects are looked up."""
    if value is None or isinstance(value, DType):
        return value
    key = str(value)
    if key.startswith("torch."):
        key = key[len("torch."):]
    try:
        return _LOOKUP[key]
    except KeyError:
        raise SpecError(f"unsupported dtype {value!r}") from None


# ----------------------------------------------------------------------------- dims
@dataclasses.dataclass(frozen=True)
class Dim:
    """A named extent; a ``dynamic`` dim is planned at ``hint`` and bound at call time."""

    name: str
    size: int | None = None
    dynamic: bool = False
    hint: int | None = None

    @property
    def extent(self) -> int:
        for candidate in (self.size, self.hint):
            if candidate is not None:
                return int(candidate)
        raise SpecError(f"dim {self.name!r} has no size; bind it (shapes={{{self.name!r}: ...}})")

    def bind(self, size) -> "Dim":
        return dataclasses.replace(self, size=None if size is None else int(size))

    def _shift(self, k):
        if isinstance(k, bool) or not isinstance(k, int):
            return NotImplemented
        moved = [None if n is None else n + k for n in (self.size, self.hint)]
        return Dim(f"{self.name}{k:+d}", moved[0], self.dynamic, moved[1])

    __add__ = __radd__ = _shift  # ``batch + 1``: the length of a CSR indptr

    def __repr__(self):
        parts = [repr(self.name)]
        if self.size is not None:
            parts.append(f"size={self.size!r}")
        if self.hint is not None:
            parts.append(f"hint={self.hint!r}")
        if self.dynamic:
            parts.append("dynamic=True")
        return f"Dim({', '.join(parts)})"


def dims(names: str, dynamic: bool = False) -> tuple:
    """``M, K = cl.dims("M K")``."""
    return tuple(Dim(n, dynamic=dynamic) for n in names.replace(",", " ").split())


def extent(d) -> int:
    return d.extent if isinstance(d, Dim) else int(d)


def dim_name(d):
    return d.name if isinstance(d, Dim) else None


# ----------------------------------------------------------------------------- annotations
@dataclasses.dataclass(frozen=True)
class TensorSpec:
    dims: tuple
    dtype: DType | None = None
    optional: bool = False  # written ``cl.Tensor[...] | None``

    def __or__(self, other):
        return dataclasses.replace(self, optional=True) if other is None else NotImplemented

    __ror__ = __or__


@dataclasses.dataclass(frozen=True)
class ScalarSpec:
    dtype: DType


class Scalar:
    """``cl.Scalar[cl.f32]``: a run-time scalar argument (paged programs)."""

    def __class_getitem__(cls, dt):
        return ScalarSpec(as_dtype(dt))


class Split:
    """A dim that may be split (split-K / split-KV) and the factors to try."""

    __slots__ = ("dim", "factors")

    def __init__(self, dim, factors=(4, 8, 16)):
        object.__setattr__(self, "dim", dim.name if isinstance(dim, Dim) else str(dim))
        object.__setattr__(self, "factors", tuple(int(f) for f in factors))

    def __setattr__(self, *_):
        raise dataclasses.FrozenInstanceError("cl.Split is immutable")

    def __eq__(self, other):
        return isinstance(other, Split) and (self.dim, self.factors) == (other.dim, other.factors)

    def __hash__(self):
        return hash((self.dim, self.factors))

    def __repr__(self):
        return f"Split({self.dim!r}, {self.factors!r})"


def _listed(split):
    if split is None or split is False:
        return ()
    return (split,) if isinstance(split, (str, Dim, Split)) else tuple(split)


def as_splits(split) -> tuple:
    return tuple(s if isinstance(s, Split) else Split(s) for s in _listed(split))


def split_names(split) -> tuple:
    """Dim names of ``"K" | Dim | Split | iterable of those``, first occurrence order."""
    names = []
    for s in _listed(split):
        n = s.dim if isinstance(s, Split) else s.name if isinstance(s, Dim) else str(s)
        if n not in names:
            names.append(n)
    return tuple(names)


def is_number(x) -> bool:
    return isinstance(x, numbers.Real) and not isinstance(x, bool)


_scalar = is_number  # the reference's private name, used by its own modules


# ----------------------------------------------------------------------------- the proxy
class Tensor:
    """Handle of one value of a program; also the annotation ``cl.Tensor["M", "K", cl.f16]``."""

    __array_priority__ = 1000

    def __class_getitem__(cls, items):
        items = items if isinstance(items, tuple) else (items,)
        dtype, shape = None, []
        for item in items:
            if isinstance(item, DType):
                dtype = item
            elif isinstance(item, str):
                shape.append(Dim(item))
            elif isinstance(item, Dim) or (isinstance(item, int) and not isinstance(item, bool)):
                shape.append(item)
            else:
                raise TypeError(f"bad cl.Tensor annotation item {item!r}")
        return TensorSpec(tuple(shape), dtype)

    def __init__(self, program, id: int, dims: tuple, dtype: DType, trans: bool = False):
        self.program = program
        self.id = id
        self.dims = tuple(dims)
        self.dtype = dtype
        self._trans = trans

    # shape
    @property
    def shape(self) -> tuple:
        return tuple(extent(d) for d in self.dims)

    @property
    def ndim(self) -> int:
        return len(self.dims)

    def __repr__(self):
        names = ", ".join(dim_name(d) or str(d) for d in self.dims)
        return f"Tensor(%{self.id}{'.mT' if self._trans else ''}[{names}] {self.dtype!r})"

    # transposed views exist only as matmul operands
    @property
    def mT(self) -> "Tensor":
        if self.ndim < 2:
            raise SpecError(".mT needs a tensor of rank >= 2")
        swapped = self.dims[:-2] + (self.dims[-1], self.dims[-2])
        return Tensor(self.program, self.id, swapped, self.dtype, not self._trans)

    @property
    def T(self) -> "Tensor":
        if self.ndim != 2:
            raise SpecError(".T is only defined for 2-D tensors; use .mT")
        return self.mT

    def view(self, *shape):
        hook = getattr(self.program, "_view", None)
        if hook is None:
            raise SpecError(".view is only lowerable inside a paged (dynamic) program")
        if len(shape) == 1 and isinstance(shape[0], tuple):
            shape = shape[0]
        return hook(self, shape)

    # arithmetic: everything is recorded by the owning builder
    def __matmul__(self, other):
        return self.program._matmul(self, other)

    def __rmatmul__(self, other):
        return self.program._matmul(other, self)

    def __add__(self, other):
        return self.program._binary("add", self, other)

    __radd__ = __add__

    def __mul__(self, other):
        return self.program._binary("mul", self, other)

    __rmul__ = __mul__

    def __truediv__(self, other):
        return self.program._binary("div", self, other)

    def __rtruediv__(self, other):
        return self.program._binary("div", other, self)

    def __neg__(self):
        return self * -1.0

    def __sub__(self, other):
        if is_number(other):
            return self + (-float(other))
        return self.program._binary("sub", self, other)

    def __rsub__(self, other):
        if is_number(other):
            return -self + float(other)
        return self.program._binary("sub", other, self)

    def __pow__(self, p):
        if p == 2:
            return self * self
        if p == 0.5:
            return self.sqrt()
        if p == -0.5:
            return self.rsqrt()
        raise SpecError(f"x ** {p!r}: only 2, 0.5 and -0.5 are lowerable")

    def exp(self):
        return self.program._unary("exp", self)

    def sqrt(self):
        return self.program._unary("sqrt", self)

    def silu(self):
        return self.program._unary("silu", self)

    def rsqrt(self):
        return 1.0 / self.sqrt()

    def _need_keepdim(self, keepdim):
        if not keepdim:
            raise SpecError("tile-IR reductions keep the reduced axis; pass keepdim=True")

    def sum(self, dim: int = -1, keepdim: bool = False):
        self._need_keepdim(keepdim)
        return self.program._reduction(self, dim)

    def max(self, dim: int = -1, keepdim: bool = False):
        self._need_keepdim(keepdim)
        hook = getattr(self.program, "_max", None)
        if hook is None:
            raise SpecError(".max is only lowerable in a dense program")
        return hook(self, dim)

    def mean(self, dim: int = -1, keepdim: bool = False):
        return self.sum(dim, keepdim) / float(self.shape[dim])

    def __bool__(self):
        raise SpecError("data-dependent control flow on a traced cl.Tensor")
