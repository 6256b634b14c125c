from __future__ import annotations

import math

from ..core.errors import LoweringRejected
from ..ir import graph as irg
from ..ir.families import Lowered, recognize


class StageGraph(irg.Graph):
    """A flat graph plus what it was recognised as and the role it plays in its variant."""

    def __init__(self, base: irg.Graph, lowered: Lowered, role: str = "main", split_factor: int | None = None,
                 placeholders=None, outputs=None):
        super().__init__(base.nodes, base.dtype, base.name)
        self.lowered = lowered
        self.role = role
        self.split_factor = split_factor
        self._phs = placeholders
        self._outs = outputs

    @property
    def placeholders(self):
        return list(self._phs) if self._phs is not None else super().placeholders

    @property
    def outputs(self):
        return list(self._outs) if self._outs is not None else super().outputs


def to_ir(structure, symbol_map=None, dtype="float16", out_dtype=None, input_names=None, name="graph"):
    """Structure -> recognised single-stage graph (role ``main``)."""
    g = irg.to_ir(structure, symbol_map, dtype, out_dtype, input_names, name)
    return StageGraph(g, recognize(g))


def partial_buffers(low: Lowered, factor: int) -> list:
    """``[(name, shape, dtype)]`` of what a split partial writes and its combine reads, split-major
    like the reference's ``(split, batch, heads[, D])`` layout
    (``python/cleave/dynamic/paging/tensor_maps.py:41-69``); f32 except the MLA value partials."""
    p = low.problem
    if low.family in ("matmul", "rmsnorm_matmul", "lora"):
        batch = max(p["batch_A"], p["batch_B"])
        bufs = [("PACC", (factor, batch * p["M"], p["N"]), "float32")]
        if low.family == "rmsnorm_matmul":
            bufs.append(("PSS", (factor, batch * p["M"]), "float32"))
        if low.family == "lora":
            bufs.append(("PD", (factor, p["M"], p["R"]), "float32"))     # partial sums of the rank-R product x @ a
        return bufs
    if low.family == "attention":
        rows, width = p["units"] * p["group"] * p["sq"], p["vdim"]
    elif low.family == "mla":
        # every split covers all heads of a batch entry, so the value partials are as large as
        # `factor` outputs: they are kept in the element type, normalised per split, with the
        # split's log-sum-exp in PM and PL = 1 (the reference's partials are in the element type too)
        rows, width = p["batch"] * p["heads"], p["ckv"]
        return [("PM", (factor, rows), "float32"), ("PL", (factor, rows), "float32"),
                ("PO", (factor, rows, width), low.dtype)]
    else:
        raise LoweringRejected(f"family {low.family!r} has no split form")
    return [("PM", (factor, rows), "float32"), ("PL", (factor, rows), "float32"),
            ("PO", (factor, rows, width), "float32")]


def _split_extent(low: Lowered) -> int:
    key = "skv" if low.family in ("attention", "mla") else "K"
    if key not in low.problem:
        raise LoweringRejected(f"family {low.family!r} has no split form")
    return low.problem[key]


def split_stages(graph: StageGraph, factor: int) -> list:
    """``[partial, combine]`` stage graphs of a recognised operator at ``factor``."""
    low = graph.lowered
    total = _split_extent(low)
    if factor < 2 or total % factor:
        raise LoweringRejected(f"split factor {factor} does not divide the split extent {total}")
    bufs = partial_buffers(low, factor)
    part_outs = [irg.OutputNode(f"OutputNode_{i}", shape, dt) for i, (_, shape, dt) in enumerate(bufs)]
    comb_ins = [irg.PlaceHolderNode(f"PlaceHolder_{n}", shape, dt) for n, shape, dt in bufs]
    if low.family == "lora":
        # the rank update happens in the combine, which therefore also reads the up factor
        comb_ins.append(low.operands["LB"])
    partial = StageGraph(graph, low, "partial", factor, outputs=part_outs)
    combine = StageGraph(graph, low, "combine", factor, placeholders=comb_ins)
    partial.name, combine.name = f"{graph.name}.partial", f"{graph.name}.combine"
    return [partial, combine]


def join_cut_pair(partial, combine) -> list:
    """One structure from an already cut ``[partial, combine]`` pair as the reference's split pass
    leaves it (``python/cleave/lower/split.py:701-717``; stored examples:
    ``tests/integration/graph_structures/*/after_split_*.graph``): both halves number their tensors
    from the same start, and the k-th output of the partial is the k-th input of the combine.  The
    halves are joined there, so that the operator is recognised as a whole and cut again into the
    partial and combine kernels this back end has for it."""
    def tensors(entry, key):
        return list(entry.get(key, ()))

    handed = [tensors(e, "input_tensors")[0] for e in partial if e["op_type"] == "kn_output_op"]
    taken = [tensors(e, "output_tensors")[0] for e in combine if e["op_type"] == "kn_input_op"]
    if len(handed) != len(taken) or not handed:
        raise LoweringRejected(f"cut pair: the partial hands over {len(handed)} tensors, the combine takes {len(taken)}")
    shift = 1 + max(t["guid"] for e in partial for key in ("input_tensors", "output_tensors") for t in tensors(e, key))
    rename = {}
    for out_t, in_t in zip(handed, taken):
        if [d for d in out_t["dim"] if d] != [d for d in in_t["dim"] if d]:
            raise LoweringRejected(f"cut pair: partial output {out_t['dim']} does not fit combine input {in_t['dim']}")
        rename[in_t["guid"]] = out_t["guid"]

    def moved(t):
        return dict(t, guid=rename.get(t["guid"], t["guid"] + shift))

    joined = [e for e in partial if e["op_type"] != "kn_output_op"]
    for e in combine:
        if e["op_type"] == "kn_input_op":
            continue
        e = dict(e)
        for key in ("input_tensors", "output_tensors"):
            if key in e:
                e[key] = [moved(t) for t in e[key]]
        joined.append(e)
    return joined


def _is_cut_pair(structure) -> bool:
    return len(structure) == 2 and all(isinstance(half, (list, tuple)) for half in structure)


def to_bundles(structures, symbol_map=None, split_factors=None, dtype="float16", out_dtype=None,
               input_names=None, **_ignored) -> list:
    """One bundle per structure: ``[main]`` or, with ``split_factors=[f]``, ``[partial, combine]``.
    A structure given as ``[partial_structure, combine_structure]`` (an already cut pair) is
    joined, recognised as one operator and cut into this back end's own stages, at
    ``split_factors[0]`` or, without it, at the split count the pair's split ops state."""
    out = []
    for s in structures:
        pair = _is_cut_pair(s)
        g = to_ir(join_cut_pair(*s) if pair else s, symbol_map, dtype, out_dtype, input_names)
        factor = int(split_factors[0]) if split_factors else None
        if pair and factor is None:
            stated = {n.shape[0] for n in g.nodes if getattr(n, "op", None) == "split"}
            if len(stated) != 1:
                raise LoweringRejected(f"cut pair: split ops state the split counts {sorted(stated)}")
            factor = stated.pop()
        out.append(split_stages(g, factor) if factor else [g])
    return out
