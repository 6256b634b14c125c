"""A light dataflow graph over the fixed op vocabulary, built from op-dict structures.

The reference's IR (``python/cleave/ir/graph.py:87-1015``) sits on TVM block analysis and
carries the whole scheduling state.  This one only has to answer "which kernel family is
this, with which operands and sizes": node shapes come straight from the structure, and
scheduling state lives in ``KernelPlan`` (``cleave_amd.schedule``), not on the graph.

Structures are lists of dicts in the superoptimizer's ``get_graph_structure()`` schema
(``python/cleave/core/schema.py``): ``op_type`` ``kn_<kind>_op``, ``input_tensors`` /
``output_tensors`` with ``dim`` (zero-padded to five entries in stored files) and ``guid``,
plus ``trans_A``/``trans_B`` on matmuls and ``scalar``/``scalar_on_left`` on scalar binaries.
"""

from __future__ import annotations

import re
from dataclasses import dataclass, field

from ..core.errors import LoweringRejected

_REDUCE = re.compile(r"^reduce_(sum|max)_(\d+)$")
_SPLIT = re.compile(r"^split_(\d+)$")


@dataclass(eq=False)
class Node:
    name: str
    shape: tuple
    dtype: str = "float16"

    def get_shape(self, _i: int = 0) -> tuple:
        return self.shape

    def get_dtype(self, _i: int = 0) -> str:
        return self.dtype


@dataclass(eq=False)
class PlaceHolderNode(Node):
    guid: int = 0


@dataclass(eq=False)
class ComputeOpNode(Node):
    op: str = ""                      # matmul add sub mul div exp sqrt silu reduce_sum reduce_max split
    inputs: list = field(default_factory=list)   # Node operands, in order
    scalar: float | None = None       # the constant operand of a scalar binary
    scalar_on_left: bool = False
    attrs: dict = field(default_factory=dict)    # dim (reduce/split), trans_A, trans_B


@dataclass(eq=False)
class OutputNode(Node):
    source: Node | None = None


class Graph:
    """Nodes in topological (structure) order."""

    def __init__(self, nodes, dtype: str = "float16", name: str = "graph"):
        self.nodes = list(nodes)
        self.dtype = dtype
        self.name = name
        self.dyn_dims: list = []

    @property
    def placeholders(self) -> list:
        return [n for n in self.nodes if isinstance(n, PlaceHolderNode)]

    @property
    def outputs(self) -> list:
        return [n for n in self.nodes if isinstance(n, OutputNode)]

    @property
    def ops(self) -> list:
        return [n for n in self.nodes if isinstance(n, ComputeOpNode)]

    def op_kinds(self) -> list:
        return [n.op for n in self.ops]

    def __repr__(self):
        return f"Graph({self.name!r}, {len(self.placeholders)} inputs, ops={self.op_kinds()}, {len(self.outputs)} outputs)"


def _shape(tensor: dict) -> tuple:
    dims = list(tensor["dim"])
    n = tensor.get("num_dims")
    if n is None:  # stored files pad with zeros instead
        while dims and dims[-1] == 0:
            dims.pop()
    else:
        dims = dims[:n]
    return tuple(int(d) for d in dims)


def to_ir(structure, symbol_map=None, dtype: str = "float16", out_dtype: str | None = None,
          input_names=None, name: str = "graph") -> Graph:
    """Build a ``Graph`` from one structure.  ``symbol_map`` maps the small symbolic extents
    of stored superoptimizer output (4, 8, 12 ...) to real sizes; ``input_names`` names the
    placeholders after the program's inputs (in input order)."""
    sym = {int(k): int(v) for k, v in (symbol_map or {}).items()}

    def real(shape):
        return tuple(sym.get(d, d) for d in shape)

    by_guid, nodes = {}, []
    names = list(input_names or [])
    n_in = n_out = 0
    for entry in structure:
        op_type = entry["op_type"]
        if not (op_type.startswith("kn_") and op_type.endswith("_op")):
            raise LoweringRejected(f"unknown op type {op_type!r}")
        kind = op_type[3:-3]
        ins = []
        for t in entry.get("input_tensors", ()):
            if t["guid"] not in by_guid:
                raise LoweringRejected(f"{op_type}: operand guid {t['guid']} is not produced earlier")
            ins.append(by_guid[t["guid"]])
        outs = entry.get("output_tensors", ())
        if kind == "input":
            t = outs[0]
            label = names[n_in] if n_in < len(names) else f"input_{t['guid']}"
            node = PlaceHolderNode(f"PlaceHolder_{label}", real(_shape(t)), t.get("dtype", dtype), guid=t["guid"])
            n_in += 1
            by_guid[t["guid"]] = node
            nodes.append(node)
            continue
        if kind == "output":
            src = ins[0]
            nodes.append(OutputNode(f"OutputNode_{n_out}", src.shape, out_dtype or dtype, source=src))
            n_out += 1
            continue
        t = outs[0]
        attrs = {}
        m = _REDUCE.match(kind)
        if m:
            kind, attrs["dim"] = f"reduce_{m.group(1)}", int(m.group(2))
            attrs["squeeze"] = bool(entry.get("squeeze_dim", False))
        m = _SPLIT.match(kind)
        if m:
            kind, attrs["dim"] = "split", int(m.group(1))
        if kind == "matmul":
            attrs["trans_A"] = bool(entry.get("trans_A", False))
            attrs["trans_B"] = bool(entry.get("trans_B", False))
        node = ComputeOpNode(f"{kind}_{t['guid']}", real(_shape(t)), dtype, op=kind, inputs=ins,
                             scalar=entry.get("scalar"), scalar_on_left=bool(entry.get("scalar_on_left", False)),
                             attrs=attrs)
        by_guid[t["guid"]] = node
        nodes.append(node)
    if not n_out:
        raise LoweringRejected("structure has no output op")
    return Graph(nodes, dtype, name)
