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


def _refuse_unread_fields(spec, optional, read):
    """A field the chosen layer ignores must still be at its default."""
    stray = []
    for f in fields(spec):
        if f.name not in optional or f.name in read:
            continue
        assert f.default is not MISSING, f"{f.name} has a default_factory and cannot be optional"
        value = getattr(spec, f.name)
        if isinstance(f.default, tuple):
            value = tuple(value)
        if value != f.default:
            stray.append(f"{f.name}={value!r}")
    if stray:
        raise InvalidSpec(f"the {spec.kind!r} layer does not read {', '.join(stray)}, so setting them "
                          "would have no effect on the emitted kernel")


def _need_ints(pairs):
    for name, value in pairs:
        if isinstance(value, bool) or not isinstance(value, int):
            raise InvalidSpec(f"{name} must be an int, got {value!r}")


def _default_pass_configs():
    return {"tl.disable_safe_memory_legalize": True}


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
        ints = [("num_qo_heads", self.num_qo_heads), ("num_kv_heads", self.num_kv_heads), ("page_size", self.page_size)]
        if self.rasterization is not None:
            ints.append(("rasterization", self.rasterization))
        _need_ints(ints)
        if self.num_qo_heads <= 0 or self.num_kv_heads <= 0:
            raise InvalidSpec(f"head counts must be positive, got {self.num_qo_heads}/{self.num_kv_heads}")
        if self.num_qo_heads % self.num_kv_heads:
            raise InvalidSpec(f"{self.num_qo_heads} query heads do not divide into {self.num_kv_heads} kv heads, "
                              "so a block's query tile would not be a whole head group")
        if self.num_kv_heads <= 1:
            raise InvalidSpec("a single kv head leaves the cache with no head axis; use the MLA layer instead")
        if self.kind != RAGGED_PREFILL_CAUSAL and self.group <= 1:
            raise InvalidSpec(f"{self.num_qo_heads} query heads over {self.num_kv_heads} kv heads leaves a group "
                              "of 1; the decode layers tile a head group of at least two rows")
        if self.kind in SLAB_KINDS:
            if self.page_size <= 1:
                raise InvalidSpec(f"page_size={self.page_size} makes the slab layer's address split degenerate; "
                                  f"use kind={PAGED_DECODE!r} for one token per page")
        elif self.page_size != 1:
            raise InvalidSpec(f"page_size={self.page_size} needs the slab access layer (kind={PAGED_DECODE_SLAB!r}) "
                              f"and its {self.last_page_len_input} input; only page_size=1 is expressible by the "
                              f"{self.kind!r} layer")
        if len(self.cache_inputs) != 2:
            raise InvalidSpec(f"expected a (K, V) cache pair, got {self.cache_inputs}")
        if self.kind not in KINDS:
            raise InvalidSpec(f"unknown access layer {self.kind!r}; expected {KINDS}")
        read = FIELDS_READ[self.kind]
        _refuse_unread_fields(self, OPTIONAL_FIELDS, read)
        names = [self.indptr_input, self.query_input, self.scale_input, *self.cache_inputs]
        names += [getattr(self, n) for n in ("index_input", "last_page_len_input", "query_indptr_input") if n in read]
        if len(set(names)) != len(names):
            raise InvalidSpec(f"input names collide: {names}")
        dims = [self.indptr_dim, self.scale_input]
        dims += [getattr(self, n) for n in ("batch_dim", "tokens_dim", "kv_tokens_dim", "pages_dim", "index_dim")
                 if n in read]
        if len(set(dims)) != len(dims):
            raise InvalidSpec(f"symbolic extent names collide: {dims}")
        if self.warp_policy not in ("rows", "cols", "even"):
            raise InvalidSpec(f"unsupported warp policy {self.warp_policy!r}")
        if tuple(self.grid_order) not in (("batch", "head"), ("head", "batch")):
            raise InvalidSpec(f"grid_order must permute ('batch', 'head'), got {self.grid_order}")
        if self.causal != (self.kind in CAUSAL_KINDS):
            raise InvalidSpec(f"causal={self.causal} does not match the {self.kind!r} layer; only the causal "
                              "prefill layers mask against the diagonal")


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
        ints = [("num_qo_heads", self.num_qo_heads), ("page_size", self.page_size),
                ("index_window_tiles", self.index_window_tiles)]
        if self.rasterization is not None:
            ints.append(("rasterization", self.rasterization))
        _need_ints(ints)
        if self.num_qo_heads < 16 or self.num_qo_heads % 16:
            raise InvalidSpec(f"{self.num_qo_heads} query heads is not a positive multiple of 16; MLA's query tile "
                              "is the head block itself, so the head count is the matrix-core M extent")
        if self.index_window_tiles < 1:
            raise InvalidSpec(f"index_window_tiles={self.index_window_tiles} leaves no window to stage")
        if self.index_window_tiles == 1 and self.prefetch:
            raise InvalidSpec("index_window_tiles=1 leaves the prefetch no next tile to read inside the window; "
                              "set prefetch=False or widen the window")
        if self.page_size != 1:
            raise InvalidSpec(f"page_size={self.page_size} would give the MLA cache a slot axis the gather does "
                              "not index; only page_size=1 is expressible here")
        if len(self.query_inputs) != 2:
            raise InvalidSpec(f"expected a (nope, pe) query pair, got {self.query_inputs}")
        if len(self.cache_inputs) != 2:
            raise InvalidSpec(f"expected a (ckv, kpe) cache pair, got {self.cache_inputs}")
        if self.warp_policy not in ("rows", "cols", "even"):
            raise InvalidSpec(f"unsupported warp policy {self.warp_policy!r}")
        if self.kind not in MLA_KINDS:
            raise InvalidSpec(f"unknown MLA access layer {self.kind!r}; expected {MLA_KINDS}")
        read = MLA_FIELDS_READ[self.kind]
        _refuse_unread_fields(self, MLA_OPTIONAL_FIELDS, read)
        names = [*self.query_inputs, *self.cache_inputs, self.index_input, self.indptr_input, self.scale_input]
        if "query_indptr_input" in read:
            names.append(self.query_indptr_input)
        if len(set(names)) != len(names):
            raise InvalidSpec(f"input names collide: {names}")
        dims = [self.pages_dim, self.indptr_dim, self.index_dim, self.scale_input,
                self.tokens_dim if "tokens_dim" in read else self.batch_dim]
        if len(set(dims)) != len(dims):
            raise InvalidSpec(f"symbolic extent names collide: {dims}")
        if self.causal != (self.kind == MLA_PAGED_PREFILL_CAUSAL):
            raise InvalidSpec(f"causal={self.causal} does not match the {self.kind!r} layer; only the causal "
                              "prefill layer masks against the diagonal")


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
        if self.split <= 1:
            raise InvalidSpec(f"a split factor of {self.split} is not a split")
        if not (1 <= self.split_step <= self.split and self.split % self.split_step == 0):
            raise InvalidSpec(f"split_step={self.split_step} does not divide split={self.split}")
        if not (1 <= self.cols <= head_dim and head_dim % self.cols == 0):
            raise InvalidSpec(f"cols={self.cols} does not divide the head dim {head_dim}")
        if self.loop_kind not in ("serial", "pipelined"):
            raise InvalidSpec(self.loop_kind)
        if self.input_scope not in ("s", "g"):
            raise InvalidSpec(self.input_scope)
