"""Every stored superoptimizer structure the reference keeps for its split pass
(``tests/integration/graph_structures/{matmul,rmsnorm_matmul,gqa}/before_split_*.graph``, held here
as data under ``tests/golden/graph_structures``): the ones its READMEs call valid are recognised as
the operator they spell, the ones they call invalid are refused.  The structures that split a
computed tensor are also run op by op in float64, as stored and after the split has been moved to
the inputs, against the closed form of the operator, which pins the interpreter and the rewrite."""

import json
from pathlib import Path

import numpy as np
import pytest

from cleave_amd.core.errors import LoweringRejected
from cleave_amd.ir import ComputeOpNode, OutputNode, PlaceHolderNode, recognize, to_ir
from cleave_amd.ir.graph import hoist_splits

STRUCT = Path(__file__).parent / "golden" / "graph_structures"
BEFORE = sorted(p.name for p in STRUCT.glob("before_split_*.graph"))
VALID = [n for n in BEFORE if "invalid" not in n]
INVALID = [n for n in BEFORE if "invalid" in n]


def stored(name, **kw):
    return to_ir(json.loads((STRUCT / name).read_text()), dtype="float16", **kw)


def _grouped(a, b):
    """Operands of a batched matmul with ranks aligned and the batch axes of the smaller one
    repeated group-wise (query head h reads kv head h // group)."""
    rank = max(a.ndim, b.ndim)
    a = a.reshape((1,) * (rank - a.ndim) + a.shape)
    b = b.reshape((1,) * (rank - b.ndim) + b.shape)
    for axis in range(rank - 2):
        if a.shape[axis] != b.shape[axis] and min(a.shape[axis], b.shape[axis]) > 1:
            if a.shape[axis] > b.shape[axis]:
                b = np.repeat(b, a.shape[axis] // b.shape[axis], axis=axis)
            else:
                a = np.repeat(a, b.shape[axis] // a.shape[axis], axis=axis)
    return a, b


def interpret(graph, feeds, check_shapes=True):
    """Outputs of ``graph`` computed one op at a time in float64; ``check_shapes`` compares every
    computed shape with the one the structure states (off when symbolic extents were mapped to
    real sizes, which maps equal numbers alike whatever they stand for)."""
    val = {}
    for n in graph.nodes:
        if isinstance(n, PlaceHolderNode):
            val[id(n)] = np.asarray(feeds[n.name], dtype=np.float64)
        elif isinstance(n, OutputNode):
            continue
        else:
            ins = [val[id(i)] for i in n.inputs]
            if n.op == "matmul":
                a, b = _grouped(*ins)
                a = np.swapaxes(a, -1, -2) if n.attrs.get("trans_A") else a
                b = np.swapaxes(b, -1, -2) if n.attrs.get("trans_B") else b
                out = a @ b
            elif n.op == "split":
                x, dim, parts = ins[0], n.attrs["dim"], n.shape[0]
                x = x.reshape(x.shape[:dim] + (parts, x.shape[dim] // parts) + x.shape[dim + 1:])
                out = np.moveaxis(x, dim, 0)
            elif n.op in ("reduce_sum", "reduce_max"):
                fold = np.sum if n.op == "reduce_sum" else np.max
                out = fold(ins[0], axis=n.attrs["dim"], keepdims=not n.attrs.get("squeeze"))
            elif n.op in ("add", "sub", "mul", "div"):
                if len(ins) == 1:
                    left, right = (n.scalar, ins[0]) if n.scalar_on_left else (ins[0], n.scalar)
                else:
                    left, right = ins
                out = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}[n.op](left, right)
            elif n.op in ("exp", "sqrt"):
                out = getattr(np, n.op)(ins[0])
            elif n.op == "rsqrt":
                out = 1.0 / np.sqrt(ins[0])
            else:
                raise AssertionError(f"op {n.op} is not part of the stored structures")
            assert not check_shapes or out.shape == tuple(n.shape), f"{n.name}: computed {out.shape}, structure says {tuple(n.shape)}"
            val[id(n)] = out
    return [val[id(o.source)] for o in graph.outputs]


@pytest.mark.parametrize("name", VALID)
def test_valid_structures_are_recognised(name):
    low = recognize(stored(name, symbol_map={12: 4096} if "rmsnorm" in name else None))
    family = "matmul" if "_matmul_split_k" in name else "rmsnorm_matmul" if "rmsnorm" in name else "attention"
    assert low.family == family
    has_split = any(n.op == "split" for n in stored(name).ops)
    assert (low.split_dim is not None) == has_split


@pytest.mark.parametrize("name", INVALID)
def test_invalid_structures_are_refused(name):
    with pytest.raises(LoweringRejected):
        recognize(stored(name, symbol_map={12: 4096} if "rmsnorm" in name else None))


def test_the_fixture_set_is_the_reference_s():
    assert len(VALID) == 11 and len(INVALID) == 14


MID_SPLIT = [f"before_split_gqa_graph_structure_valid_{i}.graph" for i in (2, 3, 4, 5)]


@pytest.mark.parametrize("name", MID_SPLIT)
def test_a_split_between_key_product_and_exponential_reads_as_split_keys(name):
    """Same operator, sizes and split axes as the structure that splits K and V themselves."""
    want = recognize(stored("before_split_gqa_graph_structure_valid_1.graph"))
    got = recognize(stored(name))
    assert got.family == "attention" and got.split_dim == "SKV" and got.problem == want.problem
    roles = {role: p.shape for role, p in got.operands.items()}
    assert roles == {role: p.shape for role, p in want.operands.items()}
    assert sorted(got.split_axes.values()) == sorted(want.split_axes.values()) == [1, 1]
    assert {got.operands["K"].name, got.operands["V"].name} == set(got.split_axes)


@pytest.mark.parametrize("name", ["before_split_gqa_graph_structure_valid_1.graph"] + MID_SPLIT)
def test_moving_the_split_to_the_inputs_keeps_the_values(name):
    graph = stored(name)
    moved = hoist_splits(graph)
    assert all(isinstance(n.inputs[0], PlaceHolderNode) for n in moved.ops if n.op == "split")
    assert [n.name for n in graph.ops] == [n.name for n in stored(name).ops], "the given graph is left as it is"
    rng = np.random.default_rng(5)
    q, k, v = (rng.standard_normal(p.shape) for p in graph.placeholders)
    feeds = dict(zip((p.name for p in graph.placeholders), (q, k, v)))
    as_stored, = interpret(graph, feeds)
    as_moved, = interpret(moved, feeds)
    np.testing.assert_allclose(as_moved, as_stored, rtol=1e-12, atol=1e-12)
    # closed form: softmax(q k^T / 8) v per query head, kv head = query head // 2 (the constant shift cancels)
    scores = np.einsum("hsd,htd->hst", q, np.repeat(k, 2, axis=0)) / 8.0
    weights = np.exp(scores - scores.max(axis=-1, keepdims=True))
    weights /= weights.sum(axis=-1, keepdims=True)
    np.testing.assert_allclose(as_stored, weights @ np.repeat(v, 2, axis=0), rtol=1e-10, atol=1e-12)


def test_a_split_does_not_move_through_a_reduction_or_a_broadcast():
    """Splitting the normalised weights would need a third kernel (the reference's "invalid 1"):
    the divisor has no key axis to split."""
    with pytest.raises(LoweringRejected, match="split of a computed tensor"):
        hoist_splits(stored("before_split_gqa_graph_structure_invalid_1.graph"))


def test_unread_producers_are_dropped_and_read_ones_kept():
    moved = hoist_splits(stored("before_split_gqa_graph_structure_valid_5.graph"))
    assert moved.op_kinds().count("matmul") == 2 and moved.op_kinds().count("exp") == 1
    both = hoist_splits(stored("before_split_gqa_graph_structure_invalid_6.graph"))
    assert both.op_kinds().count("exp") == 2        # the unsplit exponential is still read: K is consumed both ways
    assert any(isinstance(n, ComputeOpNode) and n.op == "split" for n in both.nodes)


# ---- what the reference's split pass makes of those structures (after_split_*): a [partial, combine]
# pair where it cuts, the structure itself where there is nothing to cut, an empty list where it refuses
from cleave_amd.lower import to_bundles  # noqa: E402
from cleave_amd.lower.stages import join_cut_pair  # noqa: E402

AFTER = sorted(p.name for p in STRUCT.glob("after_split_*.graph"))


def _after(name):
    return json.loads((STRUCT / name).read_text())


def _sizes(name):
    return {12: 4096} if "rmsnorm" in name else None


@pytest.mark.parametrize("name", AFTER)
def test_output_of_the_reference_s_split_pass_is_taken_as_it_comes(name):
    after, before_name = _after(name), name.replace("after_split", "before_split")
    if not after:
        assert "invalid" in name
        with pytest.raises(LoweringRejected):
            to_bundles([after])
        return
    stages, = to_bundles([after], symbol_map=_sizes(name))
    whole = recognize(stored(before_name, symbol_map=_sizes(name)))
    assert stages[0].lowered.family == whole.family and stages[0].lowered.problem == whole.problem
    if isinstance(after[0], list):
        assert [(g.role, g.split_factor) for g in stages] == [("partial", 2), ("combine", 2)]
        assert stages[0].lowered.split_dim == whole.split_dim is not None
        assert sorted(stages[0].lowered.split_axes.values()) == sorted(whole.split_axes.values())
    else:
        assert [g.role for g in stages] == ["main"] and whole.split_dim is None


def _spelling(graph):
    """Ops of a graph without names: kind, constants, attributes and operands as positions."""
    place = {id(n): ("in", k) for k, n in enumerate(graph.placeholders)}
    rows = []
    for n in graph.ops:
        attrs = {k: v for k, v in n.attrs.items() if not (k == "squeeze" and n.attrs.get("dim") != 0)}
        rows.append((n.op, n.scalar, tuple(sorted(attrs.items())), tuple(place[id(i)] for i in n.inputs), tuple(n.shape)))
        place[id(n)] = ("op", len(rows) - 1)
    return sorted(rows, key=repr)


@pytest.mark.parametrize("case", [2, 3, 4, 5])
def test_moved_splits_agree_with_the_reference_s_cut(case):
    """The reference cuts all five split-KV spellings into one and the same pair; joined again,
    that pair spells what moving the split to the inputs gives here (as multisets of ops with
    their constants, axes and shapes; operand positions are compared on the cut pair's own order)."""
    moved = hoist_splits(stored(f"before_split_gqa_graph_structure_valid_{case}.graph"))
    cut = to_ir(join_cut_pair(*_after(f"after_split_gqa_graph_structure_valid_{case}.graph")), dtype="float16")
    strip = lambda rows: sorted(((op, scalar, attrs, shape) for op, scalar, attrs, _, shape in rows), key=repr)  # noqa: E731
    assert strip(_spelling(moved)) == strip(_spelling(cut))
    split_inputs = lambda g: sorted((g.placeholders.index(n.inputs[0]), n.attrs["dim"]) for n in g.ops if n.op == "split")  # noqa: E731
    assert split_inputs(moved) == split_inputs(cut) == [(1, 1), (2, 1)]


@pytest.mark.parametrize("name", [n for n in AFTER if "invalid" not in n])
def test_a_joined_pair_computes_what_the_uncut_structure_computes(name):
    after = _after(name)
    joined = to_ir(join_cut_pair(*after) if isinstance(after[0], list) else after, dtype="float16")
    whole = stored(name.replace("after_split", "before_split"))
    rng = np.random.default_rng(11)
    values = [rng.standard_normal(p.shape) for p in whole.placeholders]
    assert [p.shape for p in joined.placeholders] == [p.shape for p in whole.placeholders]
    got, = interpret(joined, {p.name: v for p, v in zip(joined.placeholders, values)})
    want, = interpret(whole, {p.name: v for p, v in zip(whole.placeholders, values)})
    np.testing.assert_allclose(got.reshape(want.shape), want, rtol=1e-12, atol=1e-12)


def test_a_pair_whose_halves_do_not_fit_is_refused():
    partial, combine = _after("after_split_matmul_split_k_graph_structure.graph")
    with pytest.raises(LoweringRejected, match="hands over"):
        join_cut_pair(partial, _after("after_split_gqa_graph_structure_valid_1.graph")[1])
    widened = json.loads(json.dumps(combine))
    widened[0]["output_tensors"][0]["dim"][2] = 16
    with pytest.raises(LoweringRejected, match="does not fit"):
        join_cut_pair(partial, widened)


def test_graph_set_takes_cut_pairs_and_uncut_structures_alike():
    from cleave_amd.pipeline import GraphSet
    graphs = GraphSet.from_structures(None, [_after("after_split_gqa_graph_structure_valid_2.graph"),
                                             _after("after_split_gqa_graph_structure_valid_6.graph"),
                                             json.loads((STRUCT / "before_split_gqa_graph_structure_valid_4.graph").read_text())])
    assert [g.is_split for g in graphs] == [True, False, True]
    assert graphs[0].ops.count("matmul") == 2 and all(isinstance(entry, dict) for entry in graphs[0].structure)
