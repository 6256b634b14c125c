"""Helpers that drive lower -> tiling -> codegen -> compile without the search (explicit template and tiling in, callable kernel out)."""

from __future__ import annotations

from cleave_amd.codegen import HipCodeGen
from cleave_amd.lower import to_ir
from cleave_amd.lower.stages import split_stages
from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code
from cleave_amd.schedule import apply_tiling, search_tiling
from cleave_amd.schedule.hint import TileDict


def stage_graph(program):
    return to_ir(program.to_graph_structure(), dtype=program.dtype.name,
                 input_names=[s.name for s in program.inputs], name=program.name)


def source_for(program, template=None, tiling=None, split=None, rank=0):
    """HIP source of ``program`` at an explicit (template, tiling) or the ``rank``-th searched
    candidate; with ``split`` the fused partial+combine unit."""
    g = stage_graph(program)
    if split:
        part, comb = split_stages(g, split)
        if template:
            cand = TileDict(template, "partial", dict(tiling or {}), split_factor=split, flat_graph=part)
        else:
            cand = search_tiling(part, topk=rank + 1)[rank]
        return HipCodeGen().gen([apply_tiling(cand), apply_tiling(search_tiling(comb)[0])])
    if template:
        cand = TileDict(template, "main", dict(tiling or {}), flat_graph=g)
    else:
        cand = search_tiling(g, topk=rank + 1)[rank]
    return HipCodeGen().gen(apply_tiling(cand))


def kernel_for(program, **kw):
    src = source_for(program, **kw)
    loaded = _load_main_kernel_from_code(src)
    return _compile(loaded, loaded.manifest["out_idx"])
