"""The value table and op list under every traced program.

A recorder is a straight-line program in single-assignment form: ``values[i]`` is the handle of
value ``i``, ``oplist`` holds one ``Op`` per recorded call in call order, and every value remembers
the op that made it.  Dense programs and paged programs differ only in which op kinds they accept
and how they check them; the bookkeeping, the listing and the (de)serialisation live here.
"""

from __future__ import annotations

from ..core.errors import SpecError
from .tensor import Dim, Tensor, as_dtype, dim_name


class Op:
    """One recorded call.  ``args``: value numbers (int) and literal scalars (float), in operand
    order; ``outs``: the numbers of the values it defines; ``attrs``: its attributes, a tuple of
    (key, value) pairs sorted by key."""

    __slots__ = ("kind", "args", "outs", "attrs")

    def __init__(self, kind: str, args=(), outs=(), attrs=()):
        self.kind, self.args, self.outs = kind, tuple(args), tuple(outs)
        self.attrs = tuple(sorted(dict(attrs).items()))

    @property
    def out(self):
        """The value an op with one result defines (``None`` for an op that defines none)."""
        return self.outs[0] if self.outs else None

    def attr(self, key, default=None):
        return dict(self.attrs).get(key, default)

    def value_args(self) -> list:
        return [a for a in self.args if isinstance(a, int)]

    def scalar_args(self) -> list:
        return [a for a in self.args if not isinstance(a, int)]

    def __eq__(self, other):
        return isinstance(other, Op) and \
            (self.kind, self.args, self.outs, self.attrs) == (other.kind, other.args, other.outs, other.attrs)

    def __hash__(self):
        return hash((self.kind, self.args, self.outs, self.attrs))

    def __repr__(self):
        return f"Op({self.kind!r}, args={self.args!r}, outs={self.outs!r}, attrs={dict(self.attrs)!r})"


class Recorder:
    def __init__(self, name: str, dtype):
        self.name, self.dtype = name, as_dtype(dtype)
        self.values: list = []
        self.oplist: list = []
        self._maker: dict = {}

    # ---- reading
    def value(self, number: int) -> Tensor:
        return self.values[number]

    def producer(self, number: int) -> Op:
        return self._maker[number]

    def owns(self, x) -> bool:
        return isinstance(x, Tensor) and x.program is self

    def need(self, x, what: str) -> Tensor:
        """``x`` if it is a plain (not transposed-view) value of this recorder."""
        if not isinstance(x, Tensor):
            raise SpecError(f"{what}: expected a cl.Tensor, got {type(x).__name__}")
        if x.program is not self:
            raise SpecError(f"{what}: tensor belongs to another program")
        if x._trans:
            raise SpecError(f"{what} on a transposed view: .mT/.T only fold into matmul operands")
        return x

    # ---- writing
    def emit(self, kind: str, args=(), results=(), **attrs):
        """Append an op defining one value per ``(dims, dtype)`` in ``results``; returns the new
        handle, a tuple of them, or ``None`` when the op defines nothing."""
        made = []
        for shape, dtype in results:
            handle = Tensor(self, len(self.values), shape, dtype or self.dtype)
            self.values.append(handle)
            made.append(handle)
        op = Op(kind, args, [t.id for t in made], attrs)
        self.oplist.append(op)
        for handle in made:
            self._maker[handle.id] = op
        if not made:
            return None
        return made[0] if len(made) == 1 else tuple(made)

    # ---- showing
    def listing(self, header: str) -> str:
        lines = [header]
        for op in self.oplist:
            operands = ", ".join(f"%{a}" if isinstance(a, int) else repr(a) for a in op.args)
            notes = "".join(f" {k}={v!r}" for k, v in op.attrs if v is not False)
            lhs = ", ".join(f"%{o}" for o in op.outs)
            shapes = "; ".join(str([dim_name(d) or d for d in self.values[o].dims]) for o in op.outs)
            lines.append(f"  {lhs + ' = ' if lhs else ''}{op.kind}({operands}){notes}" + (f"  : {shapes}" if shapes else ""))
        return "\n".join(lines)


# ---- plain-data forms (JSON-safe) of the things a recorder holds ---------------------------------
def dim_to_doc(d):
    return int(d) if not isinstance(d, Dim) else {"name": d.name, "size": d.size, "dynamic": d.dynamic, "hint": d.hint}


def dim_from_doc(doc):
    return int(doc) if not isinstance(doc, dict) else Dim(doc["name"], doc["size"], doc["dynamic"], doc["hint"])
