"""Operator-level description of each access layer, with its self-consistency checks.

Field names, defaults and refusals follow ``python/cleave/dynamic/paging/specs.py:55-413``:
the names given here become the emitted kernel's parameter names, so they are part of the
operator's declared signature.  Knobs that only steer the reference's TileLang lowering
(``pass_configs``, ``rasterization``, ``warp_policy``) are accepted and carried but do not
change the HIP source.
"""

from __future__ import annotations

from dataclasses import MISSING, dataclass, field, fields

from .errors import InvalidSpec
from .kinds import (CAUSAL_KINDS, FIELDS_READ, KINDS, MLA_FIELDS_READ, MLA_KINDS, MLA_OPTIONAL_FIELDS,
                    MLA_PAGED_PREFILL_CAUSAL, OPTIONAL_FIELDS, PAGED_DECODE, PAGED_DECODE_SLAB,
                    RAGGED_PREFILL_CAUSAL, SLAB_KINDS)


def _fail(message):
    raise InvalidSpec(message)


def _check(rules):
    """``rules``: (holds, message) pairs in the order a reader would meet the problems; the first
    one that does not hold is reported."""
    for holds, message in rules:
        if not holds:
            _fail(message() if callable(message) else message)


def _whole_numbers(spec, names):
    for name in names:
        value = getattr(spec, name)
        if value is not None and (isinstance(value, bool) or not isinstance(value, int)):
            _fail(f"{name} must be an int, got {value!r}")


def _distinct(what, names):
    if len(set(names)) != len(names):
        _fail(f"{what} collide: {names}")


def _only_read_fields_are_set(spec, optional, read):
    """A field that the chosen access layer never looks at must be left at its default: a value
    there would silently change nothing in the kernel."""
    defaults = {f.name: f.default for f in fields(spec)}
    changed = []
    for name in optional:
        if name in read:
            continue
        assert defaults[name] is not MISSING, f"{name} needs a plain default to be optional"
        value = getattr(spec, name)
        value = tuple(value) if isinstance(defaults[name], tuple) else value
        if value != defaults[name]:
            changed.append(f"{name}={value!r}")
    if changed:
        _fail(f"the {spec.kind!r} layer does not read {', '.join(changed)}, so setting them would have no effect "
              "on the emitted kernel")


def _default_pass_configs():
    return {"tl.disable_safe_memory_legalize": True}


WARP_POLICIES = ("rows", "cols", "even")


@dataclass(frozen=True)
class PagingSpec:
    num_qo_heads: int
    num_kv_heads: int
    kind: str = PAGED_DECODE
    page_size: int = 1
    index_input: str = "KV_INDICES"
    indptr_input: str = "KV_INDPTR"
    query_indptr_input: str = "QO_INDPTR"
    last_page_len_input: str = "KV_LAST_PAGE_LEN"
    query_input: str = "Q"
    cache_inputs: tuple = ("K_CACHE", "V_CACHE")
    scale_input: str = "sm_scale"
    causal: bool = False
    emit_lse: bool = True
    batch_dim: str = "batch"
    tokens_dim: str = "total_q"
    kv_tokens_dim: str = "total_kv"
    pages_dim: str = "num_pages"
    indptr_dim: str = "len_indptr"
    index_dim: str = "n_idx"
    pass_configs: dict = field(default_factory=_default_pass_configs)
    rasterization: int | None = 1
    warp_policy: str = "cols"
    grid_order: tuple = ("batch", "head")

    @property
    def group(self) -> int:
        """Query heads per kv head: the real rows of one block's query tile."""
        return self.num_qo_heads // self.num_kv_heads

    def validate(self) -> None:
        _whole_numbers(self, ("num_qo_heads", "num_kv_heads", "page_size", "rasterization"))
        q, kv, page = self.num_qo_heads, self.num_kv_heads, self.page_size
        slab = self.kind in SLAB_KINDS
        _check([
            (q > 0 and kv > 0, f"head counts must be positive, got {q}/{kv}"),
            (kv <= 0 or q % kv == 0, f"{q} query heads do not divide into {kv} kv heads, so a block's query tile "
                                     "would not be a whole head group"),
            (kv > 1, "a single kv head leaves the cache with no head axis; use the MLA layer instead"),
            (self.kind == RAGGED_PREFILL_CAUSAL or kv <= 1 or q // kv > 1,
             f"{q} query heads over {kv} kv heads leaves a group of 1; the decode layers tile a head group of at "
             "least two rows"),
            (not slab or page > 1, f"page_size={page} makes the slab layer's address split degenerate; use "
                                   f"kind={PAGED_DECODE!r} for one token per page"),
            (slab or page == 1, f"page_size={page} needs the slab access layer (kind={PAGED_DECODE_SLAB!r}) and its "
                                f"{self.last_page_len_input} input; only page_size=1 is expressible by the "
                                f"{self.kind!r} layer"),
            (len(self.cache_inputs) == 2, f"expected a (K, V) cache pair, got {self.cache_inputs}"),
            (self.kind in KINDS, f"unknown access layer {self.kind!r}; expected {KINDS}"),
        ])
        read = FIELDS_READ[self.kind]
        _only_read_fields_are_set(self, OPTIONAL_FIELDS, read)
        per_layer = [getattr(self, n) for n in ("index_input", "last_page_len_input", "query_indptr_input") if n in read]
        _distinct("input names", [self.indptr_input, self.query_input, self.scale_input, *self.cache_inputs, *per_layer])
        extents = [getattr(self, n) for n in ("batch_dim", "tokens_dim", "kv_tokens_dim", "pages_dim", "index_dim")
                   if n in read]
        _distinct("symbolic extent names", [self.indptr_dim, self.scale_input, *extents])
        _check([
            (self.warp_policy in WARP_POLICIES, f"unsupported warp policy {self.warp_policy!r}"),
            (sorted(self.grid_order) == ["batch", "head"],
             f"grid_order must permute ('batch', 'head'), got {self.grid_order}"),
            (self.causal == (self.kind in CAUSAL_KINDS),
             f"causal={self.causal} does not match the {self.kind!r} layer; only the causal prefill layers mask "
             "against the diagonal"),
        ])


@dataclass(frozen=True)
class MLASpec:
    """Paged multi-head *latent* attention: one shared compressed cache (also the values),
    a rope cache adding a second score term, two query tensors, no kv-head axis."""

    num_qo_heads: int
    kind: str = "mla_paged_decode"
    page_size: int = 1
    index_window_tiles: int = 8
    prefetch: bool = True
    query_inputs: tuple = ("QN", "QP")
    cache_inputs: tuple = ("CKV", "KPE")
    index_input: str = "KVI"
    indptr_input: str = "KV_INDPTR"
    query_indptr_input: str = "QO_INDPTR"
    scale_input: str = "sm_scale"
    causal: bool = False
    emit_lse: bool = True
    batch_dim: str = "batch"
    tokens_dim: str = "total_q"
    pages_dim: str = "num_pages"
    indptr_dim: str = "len_indptr"
    index_dim: str = "n_idx"
    pass_configs: dict = field(default_factory=_default_pass_configs)
    rasterization: int | None = None
    warp_policy: str = "cols"

    def validate(self) -> None:
        _whole_numbers(self, ("num_qo_heads", "page_size", "index_window_tiles", "rasterization"))
        heads, window = self.num_qo_heads, self.index_window_tiles
        _check([
            (heads >= 16 and heads % 16 == 0,
             f"{heads} query heads is not a positive multiple of 16; MLA's query tile is the head block itself, so "
             "the head count is the matrix-core M extent"),
            (window >= 1, f"index_window_tiles={window} leaves no window to stage"),
            (window > 1 or not self.prefetch, "index_window_tiles=1 leaves the prefetch no next tile to read inside "
                                              "the window; set prefetch=False or widen the window"),
            (self.page_size == 1, f"page_size={self.page_size} would give the MLA cache a slot axis the gather does "
                                  "not index; only page_size=1 is expressible here"),
            (len(self.query_inputs) == 2, f"expected a (nope, pe) query pair, got {self.query_inputs}"),
            (len(self.cache_inputs) == 2, f"expected a (ckv, kpe) cache pair, got {self.cache_inputs}"),
            (self.warp_policy in WARP_POLICIES, f"unsupported warp policy {self.warp_policy!r}"),
            (self.kind in MLA_KINDS, f"unknown MLA access layer {self.kind!r}; expected {MLA_KINDS}"),
        ])
        read = MLA_FIELDS_READ[self.kind]
        _only_read_fields_are_set(self, MLA_OPTIONAL_FIELDS, read)
        row_ptr = [self.query_indptr_input] if "query_indptr_input" in read else []
        _distinct("input names", [*self.query_inputs, *self.cache_inputs, self.index_input, self.indptr_input,
                                  self.scale_input, *row_ptr])
        _distinct("symbolic extent names", [self.pages_dim, self.indptr_dim, self.index_dim, self.scale_input,
                                            self.tokens_dim if "tokens_dim" in read else self.batch_dim])
        _check([(self.causal == (self.kind == MLA_PAGED_PREFILL_CAUSAL),
                 f"causal={self.causal} does not match the {self.kind!r} layer; only the causal prefill layer masks "
                 "against the diagonal")])


@dataclass(frozen=True)
class CombineTiling:
    """Tiling of a split-KV combine body: partials folded per iteration, columns per block,
    block size.  The HIP combine kernel has one shape (a thread per four columns, 256
    threads), so only ``split`` changes the emitted code; the rest is validated and kept."""

    split: int
    split_step: int = 1
    cols: int = 128
    n_threads: int = 256
    loop_kind: str = "serial"
    loop_stages: int = 2
    input_scope: str = "g"

    def validate(self, head_dim: int) -> None:
        step, cols = self.split_step, self.cols
        _check([
            (self.split > 1, f"a split factor of {self.split} is not a split"),
            (1 <= step <= self.split and self.split % step == 0, f"split_step={step} does not divide split={self.split}"),
            (1 <= cols <= head_dim and head_dim % cols == 0, f"cols={cols} does not divide the head dim {head_dim}"),
            (self.loop_kind in ("serial", "pipelined"), f"unknown loop kind {self.loop_kind!r}"),
            (self.input_scope in ("s", "g"), f"unknown input scope {self.input_scope!r}"),
        ])
