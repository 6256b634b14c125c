"""Map a lowered ``Graph`` onto one of the kernel families the HIP templates implement.

The reference schedules any graph over its op vocabulary by generic tile propagation
(``python/cleave/schedule/tiling.py:593-882``).  This back end instead recognises whole
operators and hands each to a hand-written template, so the job here is pattern matching:

    matmul           [batched, grouped-broadcast]  A @ B with optional transposes
    rmsnorm_matmul   (x * rsqrt(mean(x^2)[+eps]) [* gamma]) @ w, in either the traced order or
                     the reordered (x [* gamma] @ w) * rsqrt(...) form the superoptimizer emits
                     (tests/integration/graph_structures/rmsnorm_matmul/*valid_1.graph)
    attention        softmax(q @ k^T * c [+ shift | - rowmax]) @ v, MHA / GQA / MQA by grouped
                     batch broadcast; the normalising division may sit before or after the
                     value product
    mla              the same with scores q @ kv^T + q_pe @ k_pe^T and values = kv

Split graphs (``kn_split_<axis>_op`` on inputs, a ``reduce_sum_0`` over the split axis later)
are read through: the family is that of the unsplit program and ``split_axes`` records which
placeholder axes were split.  Anything else is a ``LoweringRejected``.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

from ..core.errors import LoweringRejected
from .graph import ComputeOpNode, Graph, Node, OutputNode, PlaceHolderNode, hoist_splits


@dataclass
class Lowered:
    """A recognised operator: family, sizes and which placeholder plays which operand."""

    family: str                       # matmul | rmsnorm_matmul | swiglu | lora | matmul_rowsum | rowsum | attention | mla
    problem: dict                     # sizes and flags the template needs
    operands: dict                    # role -> PlaceHolderNode
    outputs: list                     # OutputNodes in order
    graph: Graph = field(repr=False, default=None)
    split_axes: dict = field(default_factory=dict)   # placeholder name -> axis that was split
    split_dim: str | None = None      # "K" (matmul families) or "SKV" (attention families)

    @property
    def dtype(self) -> str:
        return self.graph.dtype


# ----------------------------------------------------------------------------- helpers
def _is(n, op) -> bool:
    return isinstance(n, ComputeOpNode) and n.op == op


class _View:
    """Reads a graph with split ops and split-axis sums made transparent."""

    def __init__(self, graph: Graph):
        self.graph = graph
        self.split_axes = {}
        self.carries = {}  # node -> True when its value still has the leading split axis
        for n in graph.nodes:
            if isinstance(n, PlaceHolderNode):
                self.carries[n] = False
            elif isinstance(n, ComputeOpNode):
                if n.op == "split":
                    src = n.inputs[0]
                    if not isinstance(src, PlaceHolderNode):
                        raise LoweringRejected(f"split of a computed tensor ({src.name}) has no partial/combine cut")
                    if self.split_axes.get(src.name, n.attrs["dim"]) != n.attrs["dim"]:
                        raise LoweringRejected(f"input {src.name} split on two axes")
                    self.split_axes[src.name] = n.attrs["dim"]
                    self.carries[n] = True
                else:
                    flags = [self.carries[i] for i in n.inputs]
                    if self._is_split_sum(n):
                        self.carries[n] = False
                    else:
                        # an unsplit graph input next to a split operand is a broadcast over the
                        # splits (the query of a split-KV attention); an unsplit *computed* tensor
                        # there means two siblings took different sides of the cut
                        tensors_mixed = any(flags) and not all(flags) and any(
                            not f and not isinstance(i, PlaceHolderNode) for f, i in zip(flags, n.inputs))
                        if tensors_mixed and n.op in ("matmul", "add", "sub", "mul", "div"):
                            raise LoweringRejected(
                                f"{n.name} mixes a split operand with an unsplit one: the split boundary is not clear")
                        self.carries[n] = any(flags)
        # An input that is split for one consumer must be split for all of them: horizontally
        # fusable siblings have to share one splitting, or the partial kernel has no single grid.
        for n in graph.nodes:
            if isinstance(n, ComputeOpNode) and n.op != "split":
                for i in n.inputs:
                    if isinstance(i, PlaceHolderNode) and i.name in self.split_axes:
                        raise LoweringRejected(f"input {i.name} is consumed both split and unsplit ({n.name}): "
                                               "the split boundary is not clear")
        for out in graph.outputs:
            if self.carries.get(out.source):
                raise LoweringRejected("a graph output still carries the split axis (no reduction over it)")

    def _is_split_sum(self, n) -> bool:
        return _is(n, "reduce_sum") and n.attrs.get("dim") == 0 and self.carries.get(n.inputs[0], False)

    @property
    def is_split(self) -> bool:
        return bool(self.split_axes)

    def skip(self, n):
        """``n`` with split ops and split-axis sums peeled off."""
        while isinstance(n, ComputeOpNode) and (n.op == "split" or self._is_split_sum(n)):
            n = n.inputs[0]
        return n

    def ins(self, n) -> list:
        return [self.skip(i) for i in n.inputs]

    def rank_shift(self, n) -> int:
        return 1 if self.carries.get(n) else 0

    def shape(self, n) -> tuple:
        """Shape of ``n`` in the unsplit program."""
        n = self.skip(n)
        if isinstance(n, PlaceHolderNode):
            return tuple(n.shape)
        if self.carries.get(n):
            return None
        return tuple(n.shape)

    def reduce_dim(self, n) -> int:
        """Reduction axis of ``n`` expressed in the unsplit program, counted from the end."""
        rank = len(n.inputs[0].shape)
        return n.attrs["dim"] - rank  # negative index


def _scalar_chain(view, n):
    """Peel scalar multiplies/divides: ``(core, factor)`` with n = core * factor."""
    factor = 1.0
    while isinstance(n, ComputeOpNode) and n.op in ("mul", "div") and n.scalar is not None and len(n.inputs) == 1:
        if n.op == "mul":
            factor *= float(n.scalar)
        elif not n.scalar_on_left:
            factor /= float(n.scalar)
        else:
            break
        n = view.skip(n.inputs[0])
    return n, factor


def _match_rnorm(view, n):
    """``1 / sqrt(sum(x*x, -1) / K [+ eps])`` -> ``(x, K, eps)`` or None."""
    n = view.skip(n)
    if not (_is(n, "div") and n.scalar is not None and n.scalar_on_left and float(n.scalar) == 1.0):
        return None
    root = view.skip(n.inputs[0])
    if not _is(root, "sqrt"):
        return None
    ms = view.skip(root.inputs[0])
    eps = 0.0
    if _is(ms, "add") and ms.scalar is not None:
        eps = float(ms.scalar)
        ms = view.skip(ms.inputs[0])
    if not (_is(ms, "div") and ms.scalar is not None and not ms.scalar_on_left):
        return None
    count = float(ms.scalar)
    total = view.skip(ms.inputs[0])
    if not (_is(total, "reduce_sum") and view.reduce_dim(total) == -1):
        return None
    sq = view.skip(total.inputs[0])
    if not (_is(sq, "mul") and sq.scalar is None and len(sq.inputs) == 2):
        return None
    a, b = view.ins(sq)
    if a is not b or not isinstance(a, PlaceHolderNode):
        return None
    if int(count) != a.shape[-1]:
        return None
    return a, int(count), eps


def _gamma_of(view, n, x):
    """``n`` is ``x`` or ``x * gamma`` (gamma a placeholder broadcast along rows) -> gamma | False | None."""
    n = view.skip(n)
    if n is x:
        return False
    if _is(n, "mul") and n.scalar is None and len(n.inputs) == 2:
        a, b = view.ins(n)
        for u, v in ((a, b), (b, a)):
            if u is x and isinstance(v, PlaceHolderNode) and v.shape[-1] == x.shape[-1] \
                    and math.prod(v.shape) == x.shape[-1]:
                return v
    return None


# ----------------------------------------------------------------------------- families
def _try_matmul(view, out):
    mm = view.skip(out)
    if not _is(mm, "matmul"):
        return None
    a, b = view.ins(mm)
    if not (isinstance(a, PlaceHolderNode) and isinstance(b, PlaceHolderNode)):
        return None
    prob = _matmul_problem(a, b, mm.attrs["trans_A"], mm.attrs["trans_B"])
    return "matmul", prob, {"A": a, "B": b}


def _try_swiglu(view, out):
    """``(x @ w_up) * silu(x @ w_gate)`` with both products over the same activation: operands
    A (activation), B (the bare product's weight), C (the weight under the silu), the roles of
    the reference's graph (``tests/_graphs.py:403-436``)."""
    n = view.skip(out)
    if not (_is(n, "mul") and n.scalar is None and len(n.inputs) == 2):
        return None
    for up, gate in (view.ins(n), view.ins(n)[::-1]):
        if not (_is(up, "matmul") and _is(gate, "silu")):
            continue
        gmm = view.ins(gate)[0]
        if not _is(gmm, "matmul"):
            continue
        (a, b), (a2, c) = view.ins(up), view.ins(gmm)
        if a is not a2 or not all(isinstance(t, PlaceHolderNode) for t in (a, b, c)):
            continue
        if view.is_split:
            raise LoweringRejected("SwiGLU has no split-K form: the gate is not linear in its partial sums")
        if (up.attrs["trans_A"], up.attrs["trans_B"]) != (gmm.attrs["trans_A"], gmm.attrs["trans_B"]) \
                or tuple(b.shape) != tuple(c.shape):
            raise LoweringRejected("SwiGLU needs both weights in one layout")
        prob = _matmul_problem(a, b, up.attrs["trans_A"], up.attrs["trans_B"])
        if prob["batch_A"] != 1 or prob["batch_B"] != 1:
            raise LoweringRejected("SwiGLU is built for 2-D operands")
        return "swiglu", prob, {"A": a, "B": b, "C": c}
    return None


def _try_matmul_rowsum(view, out):
    """``(a @ b).sum(dim=-1)``: the row sums of a product that is never stored
    (the reference's ``tests/_graphs.py:150-160``)."""
    n = view.skip(out)
    if not (_is(n, "reduce_sum") and view.reduce_dim(n) == -1):
        return None
    mm = view.ins(n)[0]
    if not _is(mm, "matmul"):
        return None
    a, b = view.ins(mm)
    if not (isinstance(a, PlaceHolderNode) and isinstance(b, PlaceHolderNode)):
        return None
    if view.is_split:
        raise LoweringRejected("matmul + row sum has no split form here")
    prob = _matmul_problem(a, b, mm.attrs["trans_A"], mm.attrs["trans_B"])
    if prob["batch_A"] != 1 or prob["batch_B"] != 1:
        raise LoweringRejected("matmul + row sum is built for 2-D operands")
    return "matmul_rowsum", prob, {"A": a, "B": b}


def _try_lora(view, out):
    """``x @ w + (x @ la) @ lb``: a base product plus a rank-R update through a shared activation
    (the reference's ``tests/_graphs.py:438-480``): operands A (x), B (w), LA (K, R), LB (R, N)."""
    n = view.skip(out)
    if not (_is(n, "add") and n.scalar is None and len(n.inputs) == 2):
        return None
    for base, up in (view.ins(n), view.ins(n)[::-1]):
        if not (_is(base, "matmul") and _is(up, "matmul")):
            continue
        down, lb = view.ins(up)
        if not _is(down, "matmul"):
            continue
        (x, w), (x2, la) = view.ins(base), view.ins(down)
        if x is not x2 or not all(isinstance(t, PlaceHolderNode) for t in (x, w, la, lb)):
            continue
        if any(m.attrs["trans_A"] or m.attrs["trans_B"] for m in (base, up, down)):
            raise LoweringRejected("LoRA is built for row-major operands: x (M, K), w (K, N), a (K, R), b (R, N)")
        if view.is_split:
            raise LoweringRejected("LoRA has no split-K form here")
        prob = _matmul_problem(x, w, False, False)
        if prob["batch_A"] != 1 or prob["batch_B"] != 1 or len(la.shape) != 2 or len(lb.shape) != 2:
            raise LoweringRejected("LoRA is built for 2-D operands")
        if la.shape != (prob["K"], lb.shape[0]) or lb.shape[1] != prob["N"]:
            raise LoweringRejected(f"LoRA factors do not line up: a {tuple(la.shape)}, b {tuple(lb.shape)}")
        prob["R"] = int(lb.shape[0])
        return "lora", prob, {"A": x, "B": w, "LA": la, "LB": lb}
    return None


def _matmul_problem(a, b, trans_a, trans_b) -> dict:
    sa, sb = tuple(a.shape), tuple(b.shape)
    if len(sa) != len(sb) or len(sa) < 2:
        raise LoweringRejected(f"matmul operand ranks differ: {sa} vs {sb}")
    m, k = (sa[-1], sa[-2]) if trans_a else (sa[-2], sa[-1])
    k2, n = (sb[-1], sb[-2]) if trans_b else (sb[-2], sb[-1])
    if k != k2:
        raise LoweringRejected(f"matmul inner extents differ: {sa} @ {sb}")
    ba, bb = sa[:-2], sb[:-2]
    for i, (x, y) in enumerate(zip(ba, bb)):
        if x != y and i != len(ba) - 1:
            raise LoweringRejected("grouped batch broadcast is only supported on the innermost batch axis")
        if x != y and max(x, y) % min(x, y):
            raise LoweringRejected(f"batch extents {x} and {y} are not grouped-broadcastable")
    return {"M": m, "N": n, "K": k, "trans_A": bool(trans_a), "trans_B": bool(trans_b),
            "batch_A": math.prod(ba), "batch_B": math.prod(bb)}


def _try_rmsnorm_matmul(view, out):
    n = view.skip(out)
    # reordered form: (x [* gamma] @ w) * rnorm(x)
    if _is(n, "mul") and n.scalar is None and len(n.inputs) == 2:
        for mm, rn in (view.ins(n), view.ins(n)[::-1]):
            if _is(mm, "matmul"):
                hit = _match_rnorm(view, rn)
                if hit is None:
                    continue
                x, count, eps = hit
                lhs, w = view.ins(mm)
                gamma = _gamma_of(view, lhs, x)
                if gamma is None or not isinstance(w, PlaceHolderNode) or mm.attrs["trans_A"]:
                    continue
                return _norm_result(x, w, gamma, count, eps, mm)
    # traced form: ((x * rnorm(x)) [* gamma]) @ w
    if _is(n, "matmul") and not n.attrs["trans_A"]:
        lhs, w = view.ins(n)
        if not isinstance(w, PlaceHolderNode):
            return None
        gamma, core = False, lhs
        if _is(lhs, "mul") and lhs.scalar is None and len(lhs.inputs) == 2:
            a, b = view.ins(lhs)
            for u, v in ((a, b), (b, a)):
                if isinstance(v, PlaceHolderNode) and _is(u, "mul") and math.prod(v.shape) == v.shape[-1]:
                    inner = view.ins(u)
                    if any(_match_rnorm(view, t) is not None for t in inner):
                        gamma, core = v, u
        if _is(core, "mul") and core.scalar is None and len(core.inputs) == 2:
            a, b = view.ins(core)
            for x, rn in ((a, b), (b, a)):
                hit = _match_rnorm(view, rn)
                if hit is not None and hit[0] is x:
                    if gamma is not False and gamma.shape[-1] != x.shape[-1]:
                        return None
                    return _norm_result(x, w, gamma, hit[1], hit[2], n)
    return None


def _norm_result(x, w, gamma, count, eps, mm):
    if len(x.shape) != 2:
        raise LoweringRejected("fused RMSNorm->matmul is built for 2-D activations")
    prob = _matmul_problem(x, w, False, mm.attrs["trans_B"])
    prob.update(norm=True, eps=float(eps), gamma=gamma is not False)
    ops = {"A": x, "B": w}
    if gamma is not False:
        ops["GAMMA"] = gamma
    return "rmsnorm_matmul", prob, ops


def _match_scores(view, n):
    """``n`` = logits fed to exp -> dict(kind, terms=[(q, k)], scale, exact)."""
    n = view.skip(n)
    exact = False
    shift = 0.0
    if _is(n, "sub") and n.scalar is None and len(n.inputs) == 2:
        a, b = view.ins(n)
        if _is(b, "reduce_max") and view.skip(b.inputs[0]) is a and view.reduce_dim(b) == -1:
            exact, n = True, a
        else:
            return None
    elif _is(n, "add") and n.scalar is not None:
        shift, n = float(n.scalar), view.skip(n.inputs[0])
    core, scale = _scalar_chain(view, n)
    terms = []
    if _is(core, "add") and core.scalar is None and len(core.inputs) == 2:
        parts = view.ins(core)
    else:
        parts = [core]
    norms = {}
    for p in parts:
        if not (_is(p, "matmul") and not p.attrs["trans_A"] and p.attrs["trans_B"]):
            return None
        q, k = view.ins(p)
        # RMSNorm over the feature axis on either operand (QK-norm attention): x * rnorm(x)
        for side, t in (("q", q), ("k", k)):
            hit = _normed(view, t)
            if hit is not None:
                if len(parts) != 1:
                    return None
                norms[side] = hit[1]
                q, k = (hit[0], k) if side == "q" else (q, hit[0])
        if not (isinstance(q, PlaceHolderNode) and isinstance(k, PlaceHolderNode)):
            return None
        terms.append((q, k))
    return {"terms": terms, "scale": scale, "exact": exact, "shift": shift, "norms": norms}


def _normed(view, n):
    """``n`` = ``x * rnorm(x)`` for a graph input x -> ``(x, eps)`` or None."""
    n = view.skip(n)
    if not (_is(n, "mul") and n.scalar is None and len(n.inputs) == 2):
        return None
    a, b = view.ins(n)
    for x, rn in ((a, b), (b, a)):
        if isinstance(x, PlaceHolderNode):
            hit = _match_rnorm(view, rn)
            if hit is not None and hit[0] is x:
                return x, hit[2]
    return None


def _try_rowsum(view, out):
    """``x.sum(-1)`` and ``x / x.sum(-1)`` over a 2-D input (the reference's ``rowsum`` and
    ``rowsum_div`` cases, ``tests/_graphs.py:1238-1275``)."""
    n = view.skip(out)
    div = False
    if _is(n, "div") and n.scalar is None and len(n.inputs) == 2:
        x, rs = view.ins(n)
        if not (_is(rs, "reduce_sum") and view.ins(rs)[0] is x):
            return None
        div, n = True, rs
    if not (_is(n, "reduce_sum") and view.reduce_dim(n) == -1):
        return None
    x = view.ins(n)[0]
    if not isinstance(x, PlaceHolderNode):
        return None
    if view.is_split:
        raise LoweringRejected("a row reduction has no split form here")
    if len(x.shape) != 2:
        raise LoweringRejected("row reductions are built for 2-D inputs")
    return "rowsum", {"M": int(x.shape[0]), "N": int(x.shape[1]), "div": div}, {"X": x}


def _try_chained_matmul(view, out):
    """``(q @ k^T) @ v`` with nothing between the products: attention without a softmax.  It is the
    attention family with ``linear`` set: the scores themselves, rounded to the element type, weigh
    the values.  Two spellings: keys given row-major and transposed by the product (the reference's
    ``matmul_matmul_bhsd`` case, ``tests/_graphs.py:78-101``), or the middle operand given
    feature-major, ``(a @ b) @ c`` with ``b`` stored (K, N) (its ``matmul_matmul_small_k`` /
    ``_small_n`` cases, ``tests/_graphs.py:65-76``): then ``k_major`` is set as well."""
    n = view.skip(out)
    if not (_is(n, "matmul") and not n.attrs["trans_A"] and not n.attrs["trans_B"]):
        return None
    scores, v = view.ins(n)
    if not (_is(scores, "matmul") and not scores.attrs["trans_A"]):
        return None
    k_major = not scores.attrs["trans_B"]
    q, k = view.ins(scores)
    if not all(isinstance(t, PlaceHolderNode) for t in (q, k, v)):
        return None
    if view.is_split:
        raise LoweringRejected("a chained matmul has no split form here")
    sq_, sv_ = tuple(q.shape), tuple(v.shape)
    sk_ = tuple(k.shape[:-2]) + (k.shape[-1], k.shape[-2]) if k_major else tuple(k.shape)   # as (.., keys, d)
    if len(sq_) != len(sk_) or len(sq_) < 2 or sv_[:-1] != sk_[:-1] or sq_[-1] != sk_[-1]:
        raise LoweringRejected(f"chained matmul operands do not line up: {sq_}, {tuple(k.shape)}, {sv_}")
    bq, bk = sq_[:-2], sk_[:-2]
    for i, (x, y) in enumerate(zip(bq, bk)):
        if x != y and (i != len(bq) - 1 or x % y):
            raise LoweringRejected("leading extents of a chained matmul must agree (or group on the innermost one)")
    units = math.prod(bk)
    prob = {"units": units, "group": math.prod(bq) // units, "sq": sq_[-2], "skv": sk_[-2], "head_dim": sq_[-1],
            "vdim": sv_[-1], "scale": 1.0, "exact": False, "shift": 0.0, "linear": True, "k_major": k_major}
    return "attention", prob, {"Q": q, "K": k, "V": v}


def _try_attention(view, out):
    n = view.skip(out)
    value_mm = weights = denom = None
    if _is(n, "matmul"):                       # (e / sum e) @ v
        lhs, v = view.ins(n)
        if _is(lhs, "div") and lhs.scalar is None and len(lhs.inputs) == 2:
            e, s = view.ins(lhs)
            value_mm, weights, denom = n, e, s
    elif _is(n, "div") and n.scalar is None and len(n.inputs) == 2:   # (e @ v) / sum e
        num, s = view.ins(n)
        if _is(num, "matmul"):
            value_mm, weights, denom = num, view.ins(num)[0], s
    if value_mm is None or value_mm.attrs["trans_A"] or value_mm.attrs["trans_B"]:
        return None
    v = view.ins(value_mm)[1]
    if not (isinstance(v, PlaceHolderNode) and _is(weights, "exp")):
        return None
    if not (_is(denom, "reduce_sum") and view.skip(denom.inputs[0]) is weights and view.reduce_dim(denom) == -1):
        return None
    sc = _match_scores(view, weights.inputs[0])
    if sc is None:
        return None
    terms = sc["terms"]
    if len(terms) == 2:
        (q, kv), (qpe, kpe) = terms
        if kv is not v:
            (qpe, kpe), (q, kv) = terms
        if kv is not v:
            return None
        if len(q.shape) == 2 and len(kv.shape) == 2:
            # one request: q (H, D), kv (SKV, D) -- the dense body of a paged MLA operator
            prob = {"batch": 1, "heads": q.shape[0], "ckv": q.shape[1], "kpe": qpe.shape[1],
                    "skv": kv.shape[0], "scale": sc["scale"], "exact": sc["exact"], "shift": sc["shift"]}
            return "mla", prob, {"Q": q, "QPE": qpe, "KV": kv, "KPE": kpe}
        if not (len(q.shape) == 3 and len(kv.shape) == 3 and q.shape[0] == kv.shape[0]):
            raise LoweringRejected("MLA is built for q ([B,] H, D), kv ([B,] SKV, D)")
        prob = {"batch": q.shape[0], "heads": q.shape[1], "ckv": q.shape[2], "kpe": qpe.shape[2],
                "skv": kv.shape[1], "scale": sc["scale"], "exact": sc["exact"], "shift": sc["shift"]}
        return "mla", prob, {"Q": q, "QPE": qpe, "KV": kv, "KPE": kpe}
    (q, k), = terms
    sq_, sk_ = tuple(q.shape), tuple(k.shape)
    if len(sq_) != len(sk_) or len(sq_) < 2 or tuple(v.shape[:-1]) != sk_[:-1]:
        raise LoweringRejected(f"attention operands do not line up: q {sq_}, k {sk_}, v {tuple(v.shape)}")
    bq, bk = sq_[:-2], sk_[:-2]
    for i, (x, y) in enumerate(zip(bq, bk)):
        if x != y and (i != len(bq) - 1 or x % y):
            raise LoweringRejected("query heads must be a multiple of kv heads on the innermost batch axis")
    units = math.prod(bk)
    group = math.prod(bq) // units
    prob = {"units": units, "group": group, "sq": sq_[-2], "skv": sk_[-2], "head_dim": sq_[-1],
            "vdim": v.shape[-1], "scale": sc["scale"], "exact": sc["exact"], "shift": sc["shift"]}
    if sc["norms"]:
        if view.is_split:
            raise LoweringRejected("QK-norm attention has no split-KV form here")
        prob["norm_eps"] = dict(sc["norms"])      # {"q": eps, "k": eps} for the normalised operands
    return "attention", prob, {"Q": q, "K": k, "V": v}


_MATCHERS = (_try_rmsnorm_matmul, _try_swiglu, _try_lora, _try_matmul_rowsum, _try_rowsum, _try_attention,
             _try_chained_matmul, _try_matmul)


def recognize(graph: Graph) -> Lowered:
    outs = graph.outputs
    if len(outs) != 1:
        raise LoweringRejected(f"{graph.name}: kernels are built for single-output programs, got {len(outs)} outputs")
    graph = hoist_splits(graph)
    outs = graph.outputs
    view = _View(graph)
    for matcher in _MATCHERS:
        hit = matcher(view, outs[0].source)
        if hit is not None:
            family, problem, operands = hit
            used = {id(p) for p in operands.values()}
            unused = [p.name for p in graph.placeholders if id(p) not in used]
            if unused:
                raise LoweringRejected(f"{graph.name}: inputs {unused} are not part of the recognised {family}")
            split_dim = None
            if view.is_split:
                split_dim = "SKV" if family in ("attention", "mla") else "K"
                _check_split_axes(family, operands, view.split_axes)
            return Lowered(family, problem, operands, outs, graph, dict(view.split_axes), split_dim)
    raise LoweringRejected(f"{graph.name}: ops {graph.op_kinds()} match no kernel family "
                           "(matmul, rmsnorm_matmul, swiglu, lora, matmul_rowsum, rowsum, attention, mla)")


def _check_split_axes(family, operands, split_axes):
    """A split must be over the contraction (K) of a matmul family or the KV length of an
    attention family, on every operand that has that axis."""
    role_of = {p.name: r for r, p in operands.items()}
    if family in ("matmul", "rmsnorm_matmul"):
        want = {"A": 1, "B": 0}
    elif family == "attention":
        want = {"K": len(operands["K"].shape) - 2, "V": len(operands["V"].shape) - 2}
    else:
        want = {"KV": 1, "KPE": 1}
    got = {role_of[name]: axis for name, axis in split_axes.items() if name in role_of}
    for role, axis in want.items():
        if role not in got:
            raise LoweringRejected(f"split graph leaves operand {role} unsplit: the split boundary is not clear")
        if family in ("matmul", "rmsnorm_matmul"):
            continue  # transposes decide the axis; the template derives K itself
        if got[role] != axis:
            raise LoweringRejected(f"operand {role} is split on axis {got[role]}, expected the KV axis {axis}")
    extra = set(got) - set(want)
    if extra:
        raise LoweringRejected(f"operands {sorted(extra)} must not be split")
