"""Stage 1: Program -> candidate graph structures (``GraphSet``).

In the reference this stage runs the C++ algebraic superoptimizer
(``python/cleave/pipeline/superopt.py:96-127``), which this back end leaves untouched and
does not bundle.  The stage therefore proposes what the back end can consume without it:
the identity structure of the program (the reference's own ``GraphSet.identity`` fallback,
``:84-88``) and, for each requested split dim, the same structure marked split when the
recognised operator has a partial/combine form over that dim.  Structures found by the real
superoptimizer (JSON op lists) enter through ``GraphSet.from_structures``.  Results are
checkpointed under the content-addressed cache like the reference's.
"""

from __future__ import annotations

import json
import time
from dataclasses import dataclass, field
from typing import Any, Callable, Sequence

from ..core.errors import LoweringRejected, SpecError, SuperoptError
from . import cache
from .config import SuperoptConfig

_IO_OPS = ("kn_input_op", "kn_output_op")


def program_dtype(program) -> str:
    return str(getattr(program, "dtype", None) or "float16")


def _op_name(op_type: str) -> str:
    name = op_type
    if name.startswith("kn_"):
        name = name[3:]
    if name.endswith("_op"):
        name = name[:-3]
    for what in ("sum", "max"):
        if name.startswith(f"reduce_{what}"):
            return what
    return name


@dataclass(eq=False)
class SearchedGraph:
    index: int
    structure: list
    symbol_map: dict | None
    is_split: bool
    program: Any = field(repr=False, default=None)
    split: tuple = ()
    invalid_split: bool = False
    split_rejection: str | None = None

    @property
    def dtype(self) -> str:
        return program_dtype(self.program)

    @property
    def kind(self) -> str:
        if self.invalid_split:
            return "invalid-split"
        return f"split({','.join(self.split)})" if self.is_split else "solo"

    @property
    def ops(self) -> list:
        return [_op_name(o["op_type"]) for o in self.structure if o["op_type"] not in _IO_OPS]

    def summary(self) -> str:
        return f"{self.kind} " + ">".join(self.ops)

    def __repr__(self):
        return f"SearchedGraph({self.index}, {self.summary()})"


class GraphSet(Sequence):
    def __init__(self, graphs, program=None, config: SuperoptConfig | None = None, *, max_ops=None,
                 checkpoint=None, from_cache=False, seconds=0.0):
        self.graphs = list(graphs)
        self.program, self.config, self.max_ops = program, config, max_ops
        self.checkpoint, self.from_cache, self.seconds = checkpoint, from_cache, seconds

    def __len__(self):
        return len(self.graphs)

    def __getitem__(self, i):
        return self.graphs[i]

    def filter(self, fn: Callable) -> "GraphSet":
        return GraphSet([g for g in self.graphs if fn(g)], self.program, self.config, max_ops=self.max_ops,
                        checkpoint=self.checkpoint, from_cache=self.from_cache, seconds=self.seconds)

    @property
    def dtype(self) -> str:
        return program_dtype(self.program)

    @classmethod
    def identity(cls, program) -> "GraphSet":
        """The un-optimised program as its only graph."""
        return cls([SearchedGraph(0, program.to_graph_structure(), None, False, program)], program, None)

    @classmethod
    def from_structures(cls, program, structures, symbol_map=None, split=()) -> "GraphSet":
        """Wrap structures produced elsewhere (e.g. a superoptimizer checkpoint)."""
        graphs = []
        for i, s in enumerate(structures):
            has_split = any(o["op_type"].startswith("kn_split_") for o in s)
            graphs.append(SearchedGraph(i, s, symbol_map, has_split, program, tuple(split) if has_split else ()))
        return cls(graphs, program, None)

    def __str__(self):
        head = (f"GraphSet: {len(self)} graph(s) max_ops={self.max_ops} "
                f"{'cache hit' if self.from_cache else 'searched'} {self.seconds:.2f}s")
        return "\n".join([head] + [f"  {g.index}: {g.summary()}" for g in self])


def _split_dim_of(program, lowered) -> str | None:
    """Name of the program dim the recognised family can be split over (K or the KV length)."""
    from ..frontend.tensor import Dim

    if lowered.family in ("matmul", "rmsnorm_matmul", "lora"):
        node, axis = lowered.operands["A"], (-2 if lowered.problem["trans_A"] else -1)
    elif lowered.family == "attention":
        node, axis = lowered.operands["K"], (-1 if lowered.problem.get("k_major") else -2)    # feature-major keys: (d, keys)
    elif lowered.family == "mla":
        node, axis = lowered.operands["KV"], -2
    else:
        return None                     # no partial/combine form (SwiGLU: the gate is not linear)
    for spec in program.inputs:
        if f"PlaceHolder_{spec.name}" == node.name:
            d = spec.dims[axis]
            return d.name if isinstance(d, Dim) else None
    return None


def superoptimize(program, config: SuperoptConfig | None = None) -> GraphSet:
    from ..lower import to_ir

    config = config or SuperoptConfig()
    max_ops = config.resolve_max_ops(program)
    t0 = time.perf_counter()
    program.can_split(config.split)  # SpecError on a dim no input has
    ckpt, key = None, None
    if config.cache:
        key = cache.superopt_key(program, max_ops, config.split, config.concat_matmul)
        ckpt = cache.checkpoint_path(key)
        if ckpt.exists():
            try:
                stored = json.loads(ckpt.read_text())
                graphs = [SearchedGraph(g["index"], g["structure"], None, g["is_split"], program, tuple(g["split"]),
                                        g.get("invalid_split", False), g.get("split_rejection"))
                          for g in stored["graphs"]]
                return GraphSet(graphs, program, config, max_ops=max_ops, checkpoint=str(ckpt), from_cache=True,
                                seconds=time.perf_counter() - t0)
            except (OSError, ValueError, KeyError):
                pass  # a stale or partial checkpoint is recomputed
    try:
        structure = program.to_graph_structure()
        graphs = [SearchedGraph(0, structure, None, False, program)]
        if config.split:
            try:
                lowered = to_ir(structure, dtype=program_dtype(program),
                                input_names=[s.name for s in program.inputs]).lowered
                dim = _split_dim_of(program, lowered)
            except LoweringRejected as e:
                lowered, dim = None, None
                reason = str(e)
            if dim is not None and dim in config.split:
                graphs.append(SearchedGraph(1, structure, None, True, program, (dim,)))
            else:
                why = (f"the {lowered.family} family splits over {dim!r}, not {list(config.split)}"
                       if lowered is not None else reason)
                graphs.append(SearchedGraph(1, structure, None, False, program, tuple(config.split),
                                            invalid_split=True, split_rejection=why))
    except SpecError:
        raise
    except Exception as e:  # noqa: BLE001
        raise SuperoptError(f"graph proposal failed: {type(e).__name__}: {e}") from e
    if ckpt is not None:
        ckpt.write_text(json.dumps({"key": key, "graphs": [
            {"index": g.index, "structure": g.structure, "is_split": g.is_split, "split": list(g.split),
             "invalid_split": g.invalid_split, "split_rejection": g.split_rejection} for g in graphs]}))
    return GraphSet(graphs, program, config, max_ops=max_ops, checkpoint=None if ckpt is None else str(ckpt),
                    from_cache=False, seconds=time.perf_counter() - t0)
