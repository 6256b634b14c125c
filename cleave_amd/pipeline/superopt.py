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
from collections.abc import Sequence

from ..core.errors import LoweringRejected, SpecError, SuperoptError
from . import cache
from .config import SuperoptConfig

_IO_OPS = ("kn_input_op", "kn_output_op")
_GRAPH_FIELDS = ("index", "structure", "is_split", "split", "invalid_split", "split_rejection")   # what a checkpoint keeps


def program_dtype(program) -> str:
    return str(getattr(program, "dtype", None) or "float16")


def _short_op(op_type: str) -> str:
    """``kn_reduce_sum_dim1_op`` -> ``sum``, ``kn_matmul_op`` -> ``matmul``."""
    core = op_type.removeprefix("kn_").removesuffix("_op")
    for reduction in ("sum", "max"):
        if core.startswith("reduce_" + reduction):
            return reduction
    return core


class SearchedGraph:
    """One candidate structure: the op list, whether (and over which dims) it is a split form, or
    why the requested split has none."""

    __slots__ = ("index", "structure", "symbol_map", "is_split", "program", "split", "invalid_split", "split_rejection")

    def __init__(self, index, structure, symbol_map=None, is_split=False, program=None, split=(), invalid_split=False,
                 split_rejection=None):
        self.index = index
        self.structure = structure
        self.symbol_map = symbol_map
        self.is_split = bool(is_split)
        self.program = program
        self.split = tuple(split)
        self.invalid_split = bool(invalid_split)
        self.split_rejection = split_rejection

    dtype = property(lambda self: program_dtype(self.program))

    @property
    def ops(self) -> list:
        return [_short_op(entry["op_type"]) for entry in self.structure if entry["op_type"] not in _IO_OPS]

    @property
    def kind(self) -> str:
        if self.invalid_split:
            return "invalid-split"
        if self.is_split:
            return "split(" + ",".join(self.split) + ")"
        return "solo"

    def summary(self) -> str:
        return self.kind + " " + ">".join(self.ops)

    def __repr__(self):
        return f"SearchedGraph({self.index}, {self.summary()})"

    def stored(self) -> dict:
        return {name: (list(self.split) if name == "split" else getattr(self, name)) for name in _GRAPH_FIELDS}

    @classmethod
    def restored(cls, doc: dict, program) -> "SearchedGraph":
        return cls(doc["index"], doc["structure"], None, doc["is_split"], program, doc["split"],
                   doc.get("invalid_split", False), doc.get("split_rejection"))


class GraphSet(Sequence):
    """The graphs of one program, with how they were obtained."""

    def __init__(self, graphs, program=None, config: SuperoptConfig | None = None, *, max_ops=None,
                 checkpoint=None, from_cache=False, seconds=0.0):
        self.graphs = list(graphs)
        self.program = program
        self.config = config
        self.max_ops = max_ops
        self.checkpoint = checkpoint
        self.from_cache = from_cache
        self.seconds = seconds

    def __getitem__(self, position):
        return self.graphs[position]

    def __len__(self):
        return len(self.graphs)

    dtype = property(lambda self: program_dtype(self.program))

    def filter(self, keep) -> "GraphSet":
        return GraphSet(filter(keep, self.graphs), self.program, self.config, max_ops=self.max_ops,
                        checkpoint=self.checkpoint, from_cache=self.from_cache, seconds=self.seconds)

    def __str__(self):
        how = "cache hit" if self.from_cache else "searched"
        rows = [f"GraphSet: {len(self)} graph(s) max_ops={self.max_ops} {how} {self.seconds:.2f}s"]
        rows += [f"  {graph.index}: {graph.summary()}" for graph in self.graphs]
        return "\n".join(rows)

    @classmethod
    def identity(cls, program) -> "GraphSet":
        """The un-optimised program as its only graph."""
        return cls([SearchedGraph(0, program.to_graph_structure(), program=program)], program)

    @classmethod
    def from_structures(cls, program, structures, symbol_map=None, split=()) -> "GraphSet":
        """Wrap structures produced elsewhere (e.g. a superoptimizer checkpoint); a ``[partial,
        combine]`` pair left by the reference's split pass is joined into the one structure it cuts."""
        from ..lower.stages import _is_cut_pair, join_cut_pair

        def wrapped(position, structure):
            if _is_cut_pair(structure):
                structure = join_cut_pair(*structure)
            cut = any(entry["op_type"].startswith("kn_split_") for entry in structure)
            return SearchedGraph(position, structure, symbol_map, cut, program, split if cut else ())

        return cls([wrapped(i, structure) for i, structure in enumerate(structures)], program)


def _split_dim_of(program, lowered) -> str | None:
    """Name of the program dim the recognised family can be split over (K or the KV length)."""
    from ..frontend.tensor import Dim

    problem = lowered.problem
    if lowered.family in ("matmul", "rmsnorm_matmul", "lora"):
        role, axis = "A", (-2 if problem["trans_A"] else -1)
    elif lowered.family == "attention":
        role, axis = "K", (-1 if problem.get("k_major") else -2)      # feature-major keys: (d, keys)
    elif lowered.family == "mla":
        role, axis = "KV", -2
    else:
        return None                     # no partial/combine form (SwiGLU: the gate is not linear)
    wanted = lowered.operands[role].name
    for spec in program.inputs:
        if "PlaceHolder_" + spec.name == wanted:
            dim = spec.dims[axis]
            return dim.name if isinstance(dim, Dim) else None
    return None


def _proposals(program, split) -> list:
    """The identity structure, and for a requested split the same structure marked split -- or
    marked as having no split form, with the reason."""
    from ..lower import to_ir

    structure = program.to_graph_structure()
    graphs = [SearchedGraph(0, structure, program=program)]
    if not split:
        return graphs
    try:
        lowered = to_ir(structure, dtype=program_dtype(program), input_names=[spec.name for spec in program.inputs]).lowered
        dim = _split_dim_of(program, lowered)
        why = f"the {lowered.family} family splits over {dim!r}, not {list(split)}"
    except LoweringRejected as refusal:
        dim, why = None, str(refusal)
    if dim is not None and dim in split:
        graphs.append(SearchedGraph(1, structure, None, True, program, (dim,)))
    else:
        graphs.append(SearchedGraph(1, structure, program=program, split=split, invalid_split=True, split_rejection=why))
    return graphs


def _from_checkpoint(path, program):
    """The graphs a checkpoint file holds, or None (absent, stale or partial: searched again)."""
    if not path.exists():
        return None
    try:
        return [SearchedGraph.restored(doc, program) for doc in json.loads(path.read_text())["graphs"]]
    except (OSError, ValueError, KeyError):
        return None


def superoptimize(program, config: SuperoptConfig | None = None) -> GraphSet:
    config = config or SuperoptConfig()
    began = time.perf_counter()
    max_ops = config.resolve_max_ops(program)
    program.can_split(config.split)  # SpecError on a dim no input has

    def result(graphs, path, hit):
        return GraphSet(graphs, program, config, max_ops=max_ops, checkpoint=None if path is None else str(path),
                        from_cache=hit, seconds=time.perf_counter() - began)

    path, key = None, None
    if config.cache:
        key = cache.superopt_key(program, max_ops, config.split, config.concat_matmul)
        path = cache.checkpoint_path(key)
        kept = _from_checkpoint(path, program)
        if kept is not None:
            return result(kept, path, True)
    try:
        graphs = _proposals(program, tuple(config.split))
    except SpecError:
        raise
    except Exception as problem:  # noqa: BLE001
        raise SuperoptError(f"graph proposal failed: {type(problem).__name__}: {problem}") from problem
    if path is not None:
        path.write_text(json.dumps({"key": key, "graphs": [graph.stored() for graph in graphs]}))
    return result(graphs, path, False)
