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


_POINTWISE = ("add", "sub", "mul", "div", "exp", "sqrt", "rsqrt", "silu")


def _split_shape(shape, dim, factor) -> tuple:
    if shape[dim] % factor:
        raise LoweringRejected(f"extent {shape[dim]} of axis {dim} does not divide into {factor} splits")
    return (factor,) + tuple(shape[:dim]) + (shape[dim] // factor,) + tuple(shape[dim + 1:])


def hoist_splits(graph: Graph) -> Graph:
    """The same program with every split that sits on a computed tensor moved up to the graph inputs.

    The superoptimizer may place the split of a split-KV attention anywhere between the key
    product and the exponential (``tests/integration/graph_structures/gqa/*valid_{2..5}.graph``);
    everything from the keys to that point works on each key position by itself, so splitting
    the scores there and splitting the keys are one program.  A split moves through a pointwise
    op onto its tensor operand(s) of the same shape, and through a matmul onto the operand that
    owns the split axis (rows: A, columns: B).  It does not move through a reduction, a
    broadcast operand or a batch axis of a matmul: such a graph is refused.  Producers that are
    left without consumers are dropped; a producer that is still read unsplit stays, and the
    input it reads is then consumed both ways, which the family recognition refuses.  The given
    graph is left as it is."""
    if not any(n.op == "split" and isinstance(n.inputs[0], ComputeOpNode) for n in graph.ops):
        return graph
    clone = {}
    for n in graph.nodes:
        if isinstance(n, ComputeOpNode):
            clone[id(n)] = ComputeOpNode(n.name, n.shape, n.dtype, op=n.op, inputs=[clone[id(i)] for i in n.inputs],
                                         scalar=n.scalar, scalar_on_left=n.scalar_on_left, attrs=dict(n.attrs))
        elif isinstance(n, OutputNode):
            clone[id(n)] = OutputNode(n.name, n.shape, n.dtype, source=clone[id(n.source)])
        else:
            clone[id(n)] = n
    nodes = [clone[id(n)] for n in graph.nodes]
    serial = 0
    while True:
        split = next((n for n in nodes if isinstance(n, ComputeOpNode) and n.op == "split"
                      and isinstance(n.inputs[0], ComputeOpNode)), None)
        if split is None:
            break
        producer, dim, factor = split.inputs[0], split.attrs["dim"], split.shape[0]
        refusal = LoweringRejected(f"split of a computed tensor ({producer.name}) has no partial/combine cut")
        moved = []          # (operand index, axis) of the producer's operands that take the split

        if producer.op in _POINTWISE:
            for k, operand in enumerate(producer.inputs):
                if tuple(operand.shape) != tuple(producer.shape):
                    raise refusal                      # a broadcast operand: the split axis is not its own
                moved.append((k, dim))
        elif producer.op == "matmul":
            a, b = producer.inputs
            rank = len(producer.shape)
            if dim == rank - 1:
                moved.append((1, len(b.shape) - (2 if producer.attrs.get("trans_B") else 1)))
            elif dim == rank - 2:
                moved.append((0, len(a.shape) - (1 if producer.attrs.get("trans_A") else 2)))
            else:
                raise refusal
        else:
            raise refusal
        fresh, operands = [], list(producer.inputs)
        for k, axis in moved:
            serial += 1
            piece = ComputeOpNode(f"split_hoisted{serial}_{operands[k].name}", _split_shape(operands[k].shape, axis, factor),
                                  operands[k].dtype, op="split", inputs=[operands[k]], attrs={"dim": axis})
            fresh.append(piece)
            operands[k] = piece
        serial += 1
        lifted = ComputeOpNode(f"{producer.name}_hoisted{serial}", split.shape, producer.dtype, op=producer.op,
                               inputs=operands, scalar=producer.scalar, scalar_on_left=producer.scalar_on_left,
                               attrs=dict(producer.attrs))
        at = nodes.index(split)
        nodes[at:at + 1] = fresh + [lifted]
        for n in nodes:
            if isinstance(n, ComputeOpNode):
                n.inputs = [lifted if i is split else i for i in n.inputs]
            elif isinstance(n, OutputNode) and n.source is split:
                n.source = lifted
        # drop what nobody reads any more
        while True:
            read = {id(i) for n in nodes if isinstance(n, ComputeOpNode) for i in n.inputs}
            read |= {id(n.source) for n in nodes if isinstance(n, OutputNode)}
            dead = [n for n in nodes if isinstance(n, ComputeOpNode) and id(n) not in read]
            if not dead:
                break
            nodes = [n for n in nodes if not any(n is d for d in dead)]
    out = Graph(nodes, graph.dtype, graph.name)
    out.dyn_dims = list(graph.dyn_dims)
    return out
