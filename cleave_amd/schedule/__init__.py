"""Tiling search and application for gfx950.

``search_tiling(graph, topk, force_fusion, accept)`` and ``apply_tiling(cand)`` keep the
reference's entry points (``python/cleave/schedule/search.py:10-33``,
``python/cleave/schedule/tiling.py:593``); what they search and produce is specific to this
back end (see ``policy``).
"""

from __future__ import annotations

from ..core.errors import ScheduleRejected
from ..core.target import current_target
from . import policy
from .hint import TileDict
from .plan import KernelPlan, ParamSpec


def _candidates(graph, arch):
    low, role, factor = graph.lowered, graph.role, graph.split_factor
    if role == "combine":
        return policy.combine_candidates(low, factor, arch)
    fam = low.family
    if fam in ("matmul", "rmsnorm_matmul"):
        cands = []
        if policy.skinny_ok(low):
            cands += policy.skinny_candidates(low, role, factor, arch)
        if not (fam == "rmsnorm_matmul" and low.problem["trans_A"]):
            cands += policy.gemm_candidates(low, role, factor, arch)
        cands += policy.gemm_dma_candidates(low, role, factor, arch)
        if not cands:
            p = low.problem
            raise ScheduleRejected("the matmul kernels move 16-byte chunks: K % 8 == 0 (K % 64 == 0 per split when split), and the "
                                   f"extent along which each operand is contiguous a multiple of 8 (M = {p['M']}, N = {p['N']}, "
                                   f"K = {p['K']}, split = {factor or 1})")
        return cands
    if fam == "swiglu":
        cands = policy.swiglu_candidates(low, role, factor, arch)
        if not cands:
            raise ScheduleRejected("SwiGLU runs on the direct-to-LDS matmul, unsplit: K % 64 == 0 and N a multiple of half a "
                                   f"column tile (N % 16 == 0; N = {low.problem['N']}, K = {low.problem['K']})")
        return cands
    if fam == "matmul_rowsum":
        cands = policy.rowsum_candidates(low, role, factor, arch)
        if not cands:
            raise ScheduleRejected("matmul + row sum walks whole column tiles with one set of accumulators: unsplit, K % 64 == 0 "
                                   f"and N % 16 == 0 (N = {low.problem['N']}, K = {low.problem['K']})")
        return cands
    if fam == "rowsum":
        cands = policy.rowsum_only_candidates(low, role, factor, arch)
        if not cands:
            raise ScheduleRejected(f"row reductions read 16-byte chunks, unsplit: N % 8 == 0 (N = {low.problem['N']})")
        return cands
    if fam == "lora":
        cands = policy.lora_candidates(low, role, factor, arch)
        if not cands:
            raise ScheduleRejected("LoRA runs on the few-row matmul kernel only: M <= 64, K % 32 == 0, N % 8 == 0 "
                                   "(N % 256 == 0 when split), rank a multiple of 8 up to 64")
        return cands
    if fam == "attention":
        # the LDS-shared many-row kernel takes widths in 64-feature panels up to 256; the streaming kernel
        # head_dim % 32 == 0 with a value width of 64 or a multiple of 128
        many = policy.attn_many_rows_candidates(low, role, factor, arch)
        if low.problem.get("norm_eps") or low.problem.get("linear"):
            if not many:
                raise ScheduleRejected("QK-norm attention and chained matmuls run on the many-row kernel only: widths in "
                                       "64-feature panels up to 256, keys split into equal ranges (whole 32-key steps "
                                       "when feature-major)")
            return many
        cands = (policy.attn_candidates(low, role, factor, arch) if policy.attn_ok(low) else []) + many
        if not cands:
            raise ScheduleRejected(f"no attention kernel for key/value widths {low.problem['head_dim']}/{low.problem['vdim']} "
                                   f"with {low.problem['group'] * low.problem['sq']} query rows per unit: the streaming "
                                   "(decode) kernel needs head_dim % 32 == 0 and a value width of 64 or a multiple of 128 "
                                   "that fits its registers, the many-row kernel widths that are multiples of 64 up to 256")
        return cands
    if fam == "mla":
        if not policy.mla_ok(low):
            raise ScheduleRejected("MLA template needs heads % 16 == 0 and widths that are multiples of 32")
        return policy.mla_candidates(low, role, factor, arch)
    raise ScheduleRejected(f"no template for family {fam!r}")


def search_tiling(graph, topk: int = 10, force_fusion: bool = False, accept=None, arch=None):
    """Up to ``topk`` ``TileDict`` candidates for a stage graph, best modelled cost first.
    ``accept(cand) -> bool`` filters before the cut.  ``force_fusion`` is accepted for API
    compatibility: every template here is already one fused kernel."""
    arch = arch or current_target().arch
    if not hasattr(graph, "lowered"):
        raise ScheduleRejected("search_tiling needs a recognised stage graph (cleave_amd.lower.to_ir)")
    cands = _candidates(graph, arch)
    if accept is not None:
        cands = [c for c in cands if accept(c)]
    cands.sort(key=lambda c: (c.score, c.key()))
    seen, unique = set(), []
    for c in cands:
        if c.key() not in seen:
            seen.add(c.key())
            c.flat_graph = graph
            unique.append(c)
    return _cut(unique, max(1, int(topk)))


def _cut(ranked, topk):
    """The first ``topk`` of ``ranked``, except that every template in the pool keeps a share of
    the slots (best-first within its share): the cost models of different templates are not
    calibrated against each other well enough to let one of them crowd the other out."""
    templates = []
    for c in ranked:
        if c.template not in templates:
            templates.append(c.template)
    if len(templates) < 2 or len(ranked) <= topk:
        return ranked[:topk]
    share = max(1, topk // len(templates))
    keep = set()
    for t in templates:
        keep.update(id(c) for c in [c for c in ranked if c.template == t][:share])
    for c in ranked:                      # fill what is left best-first
        if len(keep) >= topk:
            break
        keep.add(id(c))
    return [c for c in ranked if id(c) in keep][:topk]


def _name(node_name: str) -> str:
    return node_name


def apply_tiling(cand: TileDict) -> KernelPlan:
    """The scheduled plan of one candidate: parameter list in call order plus template knobs."""
    from ..lower.stages import partial_buffers

    graph = cand.flat_graph
    low, role = graph.lowered, graph.role
    dtype = graph.dtype
    params, operands = [], {}
    if role in ("main", "partial"):
        by_node = {id(n): r for r, n in low.operands.items()}
        for ph in graph.placeholders:
            params.append(ParamSpec(ph.name, ph.dtype, tuple(ph.shape), "input"))
            operands[by_node[id(ph)]] = ph.name
    else:
        keep_role = {id(n): r for r, n in low.operands.items()}      # an original input a combine reads (LoRA's up factor)
        for ph in graph.placeholders:
            params.append(ParamSpec(ph.name, ph.dtype, tuple(ph.shape), "input"))
            operands[keep_role.get(id(ph), ph.name.replace("PlaceHolder_", ""))] = ph.name
    if role == "partial":
        for out, (bname, shape, dt) in zip(graph.outputs, partial_buffers(low, cand.split_factor)):
            params.append(ParamSpec(out.name, dt, tuple(shape), "output"))
            operands[bname] = out.name
    else:
        for i, out in enumerate(graph.outputs):
            params.append(ParamSpec(out.name, out.dtype, tuple(out.shape), "output"))
            operands["OUT" if i == 0 else f"OUT{i}"] = out.name
    return KernelPlan(template=cand.template, role=role, family=low.family, dtype=dtype, problem=dict(low.problem),
                      tiling=dict(cand.tiling), params=params, operands=operands, split_factor=cand.split_factor,
                      n_threads=cand.n_threads, lds_bytes=cand.lds_bytes, label=cand.label)
