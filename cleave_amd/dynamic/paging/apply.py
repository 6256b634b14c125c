"""Wrap a scheduled dense attention plan in a paged access layer.

Entry points and gates of ``python/cleave/dynamic/paging/apply.py:28-127`` and
``constraints.py:20-142``: ``apply_paging(plan, spec)`` for a single kernel,
``apply_paging_split([partial, combine], spec)`` / ``build_split_decode(spec, dense, split,
comb)`` for a split-KV pair, ``can_page`` / ``paging_accept`` as search filters.  The dense
plan contributes the tiling (waves per workgroup, 32-token steps); the spec contributes the
operator: page table, per-request lengths, run-time scale, symbolic batch.

Parameter order of the emitted kernel is the reference's
(``tests/graph/handwritten/expected_kernels/gqa_paged_decode_h32_kv8_d128_ps64.py:301-312``):
query, caches, indptr, indices, [last page len], scale, [partials], out, lse.
"""

from __future__ import annotations

import dataclasses

from dataclasses import dataclass

from ...schedule.plan import KernelPlan, ParamSpec
from .errors import NotDenseAttention, UnsupportedTiling
from .kinds import (BUILT_KINDS, CAUSAL_KINDS, MLA_PAGED_DECODE, MLA_PAGED_PREFILL_CAUSAL, PAGED_DECODE,
                    PAGED_DECODE_SLAB, RAGGED_PREFILL_CAUSAL)
from .specs import CombineTiling, MLASpec, PagingSpec

KV_STEP = 32  # tokens one wave consumes per step of the decode template


@dataclass(frozen=True)
class DenseAttention:
    """What the access layer reads off a scheduled dense attention plan
    (``python/cleave/dynamic/paging/recognize.py:20-646``)."""

    query_rows: int
    kv_tile: int
    head_dim: int
    n_threads: int
    dtype: str
    out_dtype: str
    accum_dtype: str = "float32"
    waves: int = 4
    split: int | None = None
    prefetch: int = 1
    # Non-zero: split-KV work is cut into items of at most this many pages (one wave per kv head,
    # `waves` is then the kv-head count) instead of `split` equal parts per request.  -1 lets the
    # launch choose the size from the page-table length so that one item lands on each compute unit.
    chunk_pages: int = 0
    # Fixed-split form only, 0 = off: a request's splits are spread over the XCDs and of every pair of
    # neighbouring splits the one on the even XCD takes this many thousandths of the pair's steps
    # from the other (the template's CL_SKEW).
    skew: int = 0
    # Chunked items only: the waves of a workgroup (one per kv head) meet at a barrier before every step.
    lockstep: bool = False


@dataclass(frozen=True)
class DenseMLA:
    """What the access layer reads off a scheduled dense MLA decode plan: the operator's widths;
    the paged kernel has one tiling (one wave per 16 heads and work item, 32-token steps)."""

    heads: int
    ckv: int
    kpe: int
    dtype: str
    out_dtype: str
    kv_tile: int = KV_STEP
    n_threads: int = 64
    split: int | None = None
    # split form: table entries per work item; -1 lets the launch choose the size from the
    # table length so that two items land on each compute unit
    chunk_pages: int = -1
    # images of a 32-token step a work item keeps in LDS: the rows of `stages - 1` steps are in
    # flight while one is in the matrix cores (2: two items fit a compute unit; 3, 4: a lone item
    # no longer advances one round trip to the cache per step)
    stages: int = 2
    # waves that deal a work item's steps out between them (single kernel, one token per item):
    # 2 halves the time of an item that is alone on its compute unit
    ksplit: int = 1

    @property
    def query_rows(self) -> int:
        return self.heads

    @property
    def head_dim(self) -> int:
        return self.ckv


def read_dense_mla(plan: KernelPlan) -> DenseMLA:
    if not isinstance(plan, KernelPlan) or plan.template != "mla_decode" or plan.family != "mla":
        raise NotDenseAttention("expected a scheduled dense MLA decode plan (template mla_decode)")
    p = plan.problem
    if p.get("paged"):
        raise NotDenseAttention("the plan is already paged")
    if p["batch"] != 1:
        raise NotDenseAttention("the dense body of a paged MLA operator is one request: q (H, D), kv (SKV, D)")
    return DenseMLA(heads=p["heads"], ckv=p["ckv"], kpe=p["kpe"], dtype=plan.dtype, out_dtype=plan.dtype,
                    split=plan.split_factor)


def read_dense(plan: KernelPlan, spec):
    """The dense tiling object of ``plan`` for the layer ``spec`` asks for."""
    return read_dense_mla(plan) if isinstance(spec, MLASpec) else read_dense_attention(plan)


def read_dense_attention(plan: KernelPlan) -> DenseAttention:
    if not isinstance(plan, KernelPlan) or plan.template != "attn_decode" or plan.family != "attention":
        raise NotDenseAttention("expected a scheduled dense attention plan (template attn_decode)")
    p = plan.problem
    if p.get("paged"):
        raise NotDenseAttention("the plan is already paged")
    if p["head_dim"] != p["vdim"]:
        raise NotDenseAttention(f"K width {p['head_dim']} != V width {p['vdim']}: not a GQA body")
    expect = p["head_dim"] ** -0.5
    if abs(p["scale"] - expect) > 1e-6 * expect:
        raise NotDenseAttention(f"the dense body's scale {p['scale']} is not 1/sqrt(d) = {expect}; the run-time "
                                "sm_scale replaces exactly that constant")
    rows = p["group"] * p["sq"]
    waves = int(plan.tiling.get("WAVES", 4))
    return DenseAttention(query_rows=-(-rows // 16) * 16, kv_tile=KV_STEP, head_dim=p["head_dim"],
                          n_threads=waves * 64, dtype=plan.dtype, out_dtype=plan.dtype, waves=waves,
                          split=plan.split_factor, prefetch=int(plan.tiling.get("PREFETCH", 1)),
                          skew=int(plan.tiling.get("SKEW", 0)))


def read_dense_partial(plan: KernelPlan):
    dense = read_dense_attention(plan)
    if plan.role != "partial" or not plan.split_factor:
        raise NotDenseAttention("expected the partial plan of a split pair")
    return dense, int(plan.split_factor)


def read_dense_combine(plan: KernelPlan) -> CombineTiling:
    if not isinstance(plan, KernelPlan) or plan.role != "combine" or not plan.split_factor:
        raise NotDenseAttention("expected the combine plan of a split pair")
    return CombineTiling(split=int(plan.split_factor))


def _check_tiling(spec, dense, split: bool = False) -> None:
    if isinstance(spec, MLASpec) != isinstance(dense, DenseMLA):
        raise NotDenseAttention("the spec and the dense plan are not of the same operator family (GQA vs MLA)")
    if spec.kind not in BUILT_KINDS:
        raise UnsupportedTiling(f"the {spec.kind!r} layer is not built by this back end yet "
                                f"(built: {', '.join(BUILT_KINDS)})")
    if split and spec.kind not in (PAGED_DECODE, PAGED_DECODE_SLAB, MLA_PAGED_DECODE):
        raise UnsupportedTiling(f"split-KV is a decode transformation; got the {spec.kind!r} layer")
    if spec.kind in CAUSAL_KINDS:
        if 16 % spec.group or spec.num_kv_heads > 16:
            raise UnsupportedTiling(f"the prefill tile is 16 rows = tokens x head group: the group ({spec.group}) must "
                                    "divide 16, with at most 16 kv heads (one wave each)")
    if isinstance(spec, MLASpec):
        if dense.heads != spec.num_qo_heads:
            raise UnsupportedTiling(f"the dense body has {dense.heads} heads, the spec {spec.num_qo_heads}")
        if dense.ckv % 64 or dense.kpe % 64:
            raise UnsupportedTiling(f"latent / rope widths {dense.ckv} / {dense.kpe} are not multiples of 64")
        return
    if dense.query_rows < spec.group:
        raise UnsupportedTiling(f"a block's query tile holds {dense.query_rows} rows but the head group needs "
                                f"{spec.group}; re-tile with at least {spec.group} query rows")
    if dense.head_dim % 32 or not (dense.head_dim % 128 == 0 or dense.head_dim == 64):
        raise UnsupportedTiling(f"head_dim {dense.head_dim} is not 64 or a multiple of 128")


def _paged_params(spec: PagingSpec, dense: DenseAttention):
    d, dt = dense.head_dim, dense.dtype
    b, pages = spec.batch_dim, spec.pages_dim
    ph = lambda n: f"PlaceHolder_{n}"  # noqa: E731
    params = [
        ParamSpec(ph(spec.query_input), dt, (b, spec.num_qo_heads, d), "input"),
        ParamSpec(ph(spec.cache_inputs[0]), dt, (pages, spec.page_size, spec.num_kv_heads, d), "input"),
        ParamSpec(ph(spec.cache_inputs[1]), dt, (pages, spec.page_size, spec.num_kv_heads, d), "input"),
        ParamSpec(ph(spec.indptr_input), "int32", (spec.indptr_dim,), "input"),
        ParamSpec(ph(spec.index_input), "int32", (spec.index_dim,), "input"),
    ]
    operands = {"Q": params[0].name, "K": params[1].name, "V": params[2].name,
                "INDPTR": params[3].name, "INDICES": params[4].name}
    if spec.kind == PAGED_DECODE_SLAB:
        params.append(ParamSpec(ph(spec.last_page_len_input), "int32", (b,), "input"))
        operands["LAST"] = params[-1].name
    params.append(ParamSpec(spec.scale_input, "float32", (), "scalar"))
    return params, operands


def _paged_outputs(spec: PagingSpec, dense: DenseAttention):
    outs = [ParamSpec("OutputNode_0", dense.out_dtype, (spec.batch_dim, spec.num_qo_heads, dense.head_dim), "output")]
    operands = {"OUT": "OutputNode_0"}
    if spec.emit_lse:
        outs.append(ParamSpec("OutputNode_1", "float32", (spec.batch_dim, spec.num_qo_heads), "output"))
        operands["OUT1"] = "OutputNode_1"
    return outs, operands


def _paged_problem(spec: PagingSpec, dense: DenseAttention) -> dict:
    return {"paged": True, "page_size": spec.page_size, "kv_heads": spec.num_kv_heads,
            "q_heads": spec.num_qo_heads, "group": spec.group, "sq": 1, "head_dim": dense.head_dim,
            "vdim": dense.head_dim, "emit_lse": bool(spec.emit_lse), "units": None, "skv": 0, "scale": 1.0,
            "dim_names": {"batch": spec.batch_dim, "num_pages": spec.pages_dim, "n_idx": spec.index_dim}}


def _plan(spec, dense, role, params, operands, split=None) -> KernelPlan:
    dyn = (spec.batch_dim, spec.pages_dim, spec.index_dim)
    label = f"kv={dense.kv_tile} q={dense.query_rows} thr={dense.n_threads}"
    tiling = {"WAVES": dense.waves, "PREFETCH": dense.prefetch}
    extra = {}
    if dense.chunk_pages and split:
        tiling.update(WAVES=spec.num_kv_heads, CHUNK_PAGES=dense.chunk_pages)
        if dense.lockstep and role != "combine":
            tiling["LOCKSTEP"] = 1
        extra["derived_dims"] = [("chunk_pages", chunk_pages_expr(spec, dense.chunk_pages))]
    elif dense.skew and split and split % 2 == 0 and role != "combine" \
            and (spec.num_kv_heads * (-(-dense.query_rows // 16))) % 8 == 0:
        tiling["SKEW"] = dense.skew
    return KernelPlan(template="attn_decode", role=role, family="attention", dtype=dense.dtype, extra=extra,
                      problem=_paged_problem(spec, dense), tiling=tiling, params=params,
                      operands=operands, split_factor=split, dyn_dims=dyn, n_threads=dense.n_threads, label=label)


MAX_CHUNK_PAGES = 64      # an item's page ids live in one register per lane of a wave


def chunk_pages_expr(spec, chunk_pages: int) -> str:
    """The launch-time expression for the item size: the fixed value, or for -1 the size that
    spreads the table over the machine's compute units (each request boundary adds an item)."""
    if chunk_pages > 0:
        return str(min(chunk_pages, MAX_CHUNK_PAGES))
    from ...core.target import current_target

    cus = current_target().arch.compute_units
    return (f"max(1, min({MAX_CHUNK_PAGES}, ceildiv({spec.index_dim}, "
            f"max(1, {cus} - {spec.batch_dim}))))")


# ----------------------------------------------------------------------------- causal prefill
# Parameter order of the reference's operators (``python/cleave/dynamic/reference.py:204-278``):
# q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, sm_scale (token table) or
# q, k, v, qo_indptr, kv_indptr, sm_scale (packed keys); then out (total_q, heads, d), lse.
def _prefill_plan(spec: PagingSpec, dense: DenseAttention, shared: bool | None = None, knobs=None) -> KernelPlan:
    """``shared``: the kernel whose four waves share every key tile through LDS (128 query rows per
    workgroup, for long requests) instead of the one-wave-per-kv-head kernel with 16-row items;
    None: follow the dense tiling (four or more waves ask for the shared form).  ``knobs``: further
    tiling entries of the shared kernel (each becomes a ``CL_PF_<name>`` definition)."""
    d, dt = dense.head_dim, dense.dtype
    if shared is None:
        shared = dense.waves >= 4 and d % 64 == 0
    ragged = spec.kind == RAGGED_PREFILL_CAUSAL
    tq = spec.tokens_dim
    ph = lambda n: f"PlaceHolder_{n}"  # noqa: E731
    kv_shape = (spec.kv_tokens_dim, spec.num_kv_heads, d) if ragged else (spec.pages_dim, 1, spec.num_kv_heads, d)
    params = [
        ParamSpec(ph(spec.query_input), dt, (tq, spec.num_qo_heads, d), "input"),
        ParamSpec(ph(spec.cache_inputs[0]), dt, kv_shape, "input"),
        ParamSpec(ph(spec.cache_inputs[1]), dt, kv_shape, "input"),
        ParamSpec(ph(spec.query_indptr_input), "int32", (spec.indptr_dim,), "input"),
        ParamSpec(ph(spec.indptr_input), "int32", (spec.indptr_dim,), "input"),
    ]
    operands = {"Q": params[0].name, "K": params[1].name, "V": params[2].name, "QINDPTR": params[3].name,
                "INDPTR": params[4].name}
    if not ragged:
        params.append(ParamSpec(ph(spec.index_input), "int32", (spec.index_dim,), "input"))
        operands["INDICES"] = params[-1].name
    params.append(ParamSpec(spec.scale_input, "float32", (), "scalar"))
    outs = [ParamSpec("OutputNode_0", dense.out_dtype, (tq, spec.num_qo_heads, d), "output")]
    operands["OUT"] = "OutputNode_0"
    if spec.emit_lse:
        outs.append(ParamSpec("OutputNode_1", "float32", (tq, spec.num_qo_heads), "output"))
        operands["OUT1"] = "OutputNode_1"
    # kernel-side names of the run-time extents: the key count is the table length or the packed
    # key rows; the request count follows from the row pointers
    dim_names = {"total_q": tq, "n_idx": spec.kv_tokens_dim} if ragged else \
        {"total_q": tq, "num_pages": spec.pages_dim, "n_idx": spec.index_dim}
    problem = {"paged": True, "prefill": True, "ragged": ragged, "kv_heads": spec.num_kv_heads,
               "q_heads": spec.num_qo_heads, "group": spec.group, "head_dim": d, "vdim": d,
               "emit_lse": bool(spec.emit_lse), "units": None, "skv": 0, "sq": 0, "scale": 1.0, "dim_names": dim_names}
    threads, rows = (256, 128) if shared else (spec.num_kv_heads * 64, 16)
    return KernelPlan(template="attn_prefill", role="main", family="attention", dtype=dense.dtype,
                      extra={"derived_dims": [("batch", f"{spec.indptr_dim} - 1")]}, problem=problem,
                      tiling={"SHARED": int(bool(shared)), **(dict(knobs or {}) if shared else {})}, params=params + outs, operands=operands, split_factor=None,
                      dyn_dims=tuple(dim_names.values()), n_threads=threads, label=f"kv={KV_STEP} q={rows} thr={threads}")


def prefill_variants(plan: KernelPlan, spec) -> list:
    """Both kernels of a causal prefill layer at ``plan``'s dense tiling (the search times each)."""
    dense = read_dense_attention(plan)
    _check_tiling(spec, dense)
    return [_prefill_plan(spec, dense, shared=s) for s in ((False, True) if dense.head_dim % 64 == 0 else (False,))]


# ----------------------------------------------------------------------------- paged MLA decode
# Parameter order of the reference's operator (``python/cleave/dynamic/reference.py:282-295``):
# q_nope, q_pe, ckv_cache, kpe_cache, kv_indptr, kv_indices, sm_scale, [partials], out, lse.
def _mla_rows_dim(spec: MLASpec) -> str:
    """Extent of the query / output row axis: requests (decode) or packed query tokens (prefill)."""
    return spec.tokens_dim if spec.kind == MLA_PAGED_PREFILL_CAUSAL else spec.batch_dim


def _mla_params(spec: MLASpec, dense: DenseMLA):
    """Decode: q_nope, q_pe, ckv_cache, kpe_cache, kv_indptr, kv_indices, sm_scale; the causal
    prefill operator has qo_indptr before kv_indptr (``python/cleave/dynamic/reference.py:324-339``)."""
    dt, b, pages = dense.dtype, _mla_rows_dim(spec), spec.pages_dim
    ph = lambda n: f"PlaceHolder_{n}"  # noqa: E731
    params = [
        ParamSpec(ph(spec.query_inputs[0]), dt, (b, spec.num_qo_heads, dense.ckv), "input"),
        ParamSpec(ph(spec.query_inputs[1]), dt, (b, spec.num_qo_heads, dense.kpe), "input"),
        ParamSpec(ph(spec.cache_inputs[0]), dt, (pages, spec.page_size, dense.ckv), "input"),
        ParamSpec(ph(spec.cache_inputs[1]), dt, (pages, spec.page_size, dense.kpe), "input"),
    ]
    operands = {"Q": params[0].name, "QPE": params[1].name, "KV": params[2].name, "KPE": params[3].name}
    if spec.kind == MLA_PAGED_PREFILL_CAUSAL:
        params.append(ParamSpec(ph(spec.query_indptr_input), "int32", (spec.indptr_dim,), "input"))
        operands["QINDPTR"] = params[-1].name
    params += [ParamSpec(ph(spec.indptr_input), "int32", (spec.indptr_dim,), "input"),
               ParamSpec(ph(spec.index_input), "int32", (spec.index_dim,), "input"),
               ParamSpec(spec.scale_input, "float32", (), "scalar")]
    operands.update(INDPTR=params[-3].name, INDICES=params[-2].name)
    return params, operands


def _mla_outputs(spec: MLASpec, dense: DenseMLA):
    rows = _mla_rows_dim(spec)
    outs = [ParamSpec("OutputNode_0", dense.out_dtype, (rows, spec.num_qo_heads, dense.ckv), "output")]
    operands = {"OUT": "OutputNode_0"}
    if spec.emit_lse:
        outs.append(ParamSpec("OutputNode_1", "float32", (rows, spec.num_qo_heads), "output"))
        operands["OUT1"] = "OutputNode_1"
    return outs, operands


def mla_chunk_pages_expr(spec: MLASpec, chunk_pages: int) -> str:
    """Launch-time item size of the split form: the fixed value, or for -1 the size that puts about
    two items on every compute unit (two one-wave workgroups fit one), at least one 32-token step."""
    if chunk_pages > 0:
        return str(chunk_pages)
    from ...core.target import current_target

    cus = current_target().arch.compute_units
    return f"max(32, min(512, ceildiv({spec.index_dim}, max(1, {2 * cus} - {spec.batch_dim}))))"


def _mla_plan(spec: MLASpec, dense: DenseMLA, role, params, operands, split=None, tok: int = 1) -> KernelPlan:
    prefill = spec.kind == MLA_PAGED_PREFILL_CAUSAL
    dim_names = {"total_q": spec.tokens_dim, "num_pages": spec.pages_dim, "n_idx": spec.index_dim} if prefill else \
        {"batch": spec.batch_dim, "num_pages": spec.pages_dim, "n_idx": spec.index_dim}
    dyn = tuple(dim_names.values())
    problem = {"paged": True, "prefill": prefill, "page_size": spec.page_size, "heads": spec.num_qo_heads,
               "ckv": dense.ckv, "kpe": dense.kpe, "emit_lse": bool(spec.emit_lse), "batch": None, "skv": 0, "scale": 1.0,
               "dim_names": dim_names}
    tiling, extra = {}, {}
    if prefill:     # the request count follows from the row pointers
        extra["derived_dims"] = [("batch", f"{spec.indptr_dim} - 1")]
        tiling["TOK"] = int(tok)          # query tokens (= waves) per work item
    if split:
        tiling["CHUNK_PAGES"] = dense.chunk_pages
        extra["derived_dims"] = [("chunk_pages", mla_chunk_pages_expr(spec, dense.chunk_pages))]
    if dense.stages != 2:
        tiling["STAGES"] = int(dense.stages)
    if dense.ksplit != 1 and not split:
        tiling["KSPLIT"] = int(dense.ksplit)
    threads = dense.n_threads * max(int(tok) if prefill else 1, int(tiling.get("KSPLIT", 1)))
    label = f"kv={dense.kv_tile} q={dense.heads * (int(tok) if prefill else 1)} thr={threads}"
    if dense.stages != 2:
        label += f" stages={dense.stages}"
    if tiling.get("KSPLIT"):
        label += f" ksplit={dense.ksplit}"
    return KernelPlan(template="mla_decode", role=role, family="mla", dtype=dense.dtype, extra=extra, problem=problem,
                      tiling=tiling, params=params, operands=operands, split_factor=split, dyn_dims=dyn,
                      n_threads=threads, label=label)


def _mla_split_decode(spec: MLASpec, dense: DenseMLA, split: int) -> list:
    if dense.chunk_pages == 0 or dense.chunk_pages < -1:
        raise UnsupportedTiling("the split form of paged MLA decode cuts the token table into items: chunk_pages "
                                "must be positive or -1 (chosen at launch)")
    params, operands = _mla_params(spec, dense)
    b, h, d = spec.batch_dim, spec.num_qo_heads, dense.ckv
    items = f"ceildiv({spec.index_dim}, chunk_pages) + {b}"
    bufs = [("PM", (items, h)), ("PL", (items, h)), ("PO", (items, h, d))]
    part_outs = [ParamSpec(f"OutputNode_{i}", "float32", shape, "output") for i, (_, shape) in enumerate(bufs)]
    part_ops = {**operands, **{name: p.name for (name, _), p in zip(bufs, part_outs)}}
    partial = _mla_plan(spec, dense, "partial", params + part_outs, part_ops, split)
    comb_ins = [ParamSpec(f"PlaceHolder_{name}", "float32", shape, "input") for name, shape in bufs]
    outs, out_ops = _mla_outputs(spec, dense)
    indptr = next(q for q in params if q.name == operands["INDPTR"])
    comb_ops = {**{name: p.name for (name, _), p in zip(bufs, comb_ins)}, **out_ops, "INDPTR": indptr.name}
    combine = _mla_plan(spec, dense, "combine", comb_ins + [indptr] + outs, comb_ops, split)
    return [partial, combine]


def mla_prefill_variants(plan: KernelPlan, spec) -> list:
    """The paged MLA causal prefill kernel with two, four and one query tokens per work item and
    two to four images of a step in LDS (the search times each: an item's waves share its key
    images, which divides the traffic into the CU and raises the number of waves a CU holds, but
    they also share the LDS bandwidth that bounds this kernel's matrix work; more images keep the
    rows of more steps in flight, which a lone item needs and many resident items do not)."""
    return [apply_paging(plan, spec, tok=t, stages=s, ksplit=k)
            for t, s, k in ((2, 2, 1), (2, 3, 1), (2, 4, 1), (4, 2, 1), (4, 4, 1), (1, 2, 1), (1, 3, 1), (1, 2, 2))]


def mla_decode_variants(plan: KernelPlan, spec) -> list:
    """The paged MLA decode kernel with two and three images of a step in LDS, and with two waves
    dealing a request's steps out between them."""
    return [apply_paging(plan, spec, stages=s, ksplit=k) for s, k in ((2, 1), (3, 1), (2, 2))]


def apply_paging(plan: KernelPlan, spec, tok: int = 2, stages: int = 2, ksplit: int = 1) -> KernelPlan:
    """A single paged kernel at ``plan``'s tiling (``tok``: query tokens per work item of the
    paged MLA causal prefill layer; ``stages``: images of a step the paged MLA kernels keep in LDS;
    ``ksplit``: waves that deal an item's steps out between them)."""
    spec.validate()
    if isinstance(spec, MLASpec):
        dense = dataclasses.replace(read_dense_mla(plan), stages=int(stages), ksplit=int(ksplit))
        if ksplit > 1:
            tok = 1
        _check_tiling(spec, dense)
        params, operands = _mla_params(spec, dense)
        outs, out_ops = _mla_outputs(spec, dense)
        return _mla_plan(spec, dense, "main", params + outs, {**operands, **out_ops}, tok=tok)
    dense = read_dense_attention(plan)
    _check_tiling(spec, dense)
    if spec.kind in CAUSAL_KINDS:
        return _prefill_plan(spec, dense)
    params, operands = _paged_params(spec, dense)
    outs, out_ops = _paged_outputs(spec, dense)
    return _plan(spec, dense, "main", params + outs, {**operands, **out_ops})


def build_split_decode(spec, dense: DenseAttention, split: int, comb: CombineTiling) -> list:
    """``[partial, combine]`` paged plans for a split-KV decode; ``HipCodeGen().gen`` fuses them
    into one source with two kernels sharing the partial buffers."""
    spec.validate()
    if comb.split != split:
        raise UnsupportedTiling(f"the combine tiling is for {comb.split} splits but the partial makes {split}")
    comb.validate(dense.head_dim)
    _check_tiling(spec, dense, split=True)
    if isinstance(spec, MLASpec):
        return _mla_split_decode(spec, dense, split)
    params, operands = _paged_params(spec, dense)
    b, h, d = spec.batch_dim, spec.num_qo_heads, dense.head_dim
    # split-major partials: one request's splits sit one stride apart
    # (python/cleave/dynamic/paging/tensor_maps.py:41-69)
    if dense.chunk_pages:
        if dense.chunk_pages < -1 or dense.chunk_pages > MAX_CHUNK_PAGES or dense.query_rows > 16 \
                or spec.num_kv_heads > 16:
            raise UnsupportedTiling(f"chunked items need chunk_pages in 1..{MAX_CHUNK_PAGES} (or -1), one 16-row "
                                    "query tile and at most 16 kv heads")
        # one partial per work item: a new item at every chunk_pages table entries and every request
        items = f"ceildiv({spec.index_dim}, chunk_pages) + {b}"
        bufs = [("PM", (items, h)), ("PL", (items, h)), ("PO", (items, h, d))]
    else:
        bufs = [("PM", (split, b, h)), ("PL", (split, b, h)), ("PO", (split, b, h, d))]
    part_outs = [ParamSpec(f"OutputNode_{i}", "float32", shape, "output") for i, (_, shape) in enumerate(bufs)]
    part_ops = {**operands, **{name: p.name for (name, _), p in zip(bufs, part_outs)}}
    partial = _plan(spec, dense, "partial", params + part_outs, part_ops, split)
    comb_ins = [ParamSpec(f"PlaceHolder_{name}", "float32", shape, "input") for name, shape in bufs]
    outs, out_ops = _paged_outputs(spec, dense)
    comb_ops = {**{name: p.name for (name, _), p in zip(bufs, comb_ins)}, **out_ops}
    if dense.chunk_pages:         # the combine finds a request's items from the page-table offsets
        indptr = next(q for q in params if q.name == operands["INDPTR"])
        comb_ins.append(indptr)
        comb_ops["INDPTR"] = indptr.name
    combine = _plan(spec, dense, "combine", comb_ins + outs, comb_ops, split)
    return [partial, combine]


def apply_paging_split(plans, spec) -> list:
    if len(plans) != 2:
        raise NotDenseAttention(f"expected a [partial, combine] pair, got {len(plans)} plans")
    partial, combine = plans
    spec.validate()
    if isinstance(spec, MLASpec):
        dense = read_dense_mla(partial)
        if partial.role != "partial" or not partial.split_factor:
            raise NotDenseAttention("expected the partial plan of a split pair")
        comb = read_dense_combine(combine)
        return build_split_decode(spec, dense, int(partial.split_factor), comb)
    dense, split = read_dense_partial(partial)
    comb = read_dense_combine(combine)
    if comb.split != split:
        raise NotDenseAttention(f"the partial makes {split} splits but the combine sums {comb.split}")
    return build_split_decode(spec, dense, split, comb)


def can_page(plan, spec) -> bool:
    from ...core.errors import PagingRefusal

    try:
        spec.validate()
        _check_tiling(spec, read_dense(plan, spec))
    except PagingRefusal:
        return False
    return True


def paging_accept(spec):
    """A ``search_tiling(accept=...)`` filter: apply the candidate, then ``can_page`` it."""
    from ...schedule import apply_tiling

    def accept(cand) -> bool:
        try:
            return can_page(apply_tiling(cand), spec)
        except Exception:  # noqa: BLE001 - a filter answers, it does not stop the search
            return False

    return accept
