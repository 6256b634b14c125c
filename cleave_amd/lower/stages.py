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
    return low.problem["skv"] if low.family in ("attention", "mla") else low.problem["K"]


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


def to_bundles(structures, symbol_map=None, split_factors=None, dtype="float16", out_dtype=None,
               input_names=None, **_ignored) -> list:
    """One bundle per structure: ``[main]`` or, with ``split_factors=[f]``, ``[partial, combine]``.
    A structure given as ``[partial_structure, combine_structure]`` (an already cut pair from a
    stored file) is recognised from its partial side only when it is a plain split of a known
    family; otherwise it is refused."""
    out = []
    for s in structures:
        g = to_ir(s, symbol_map, dtype, out_dtype, input_names)
        if split_factors:
            out.append(split_stages(g, int(split_factors[0])))
        else:
            out.append([g])
    return out
