"""Shipped dynamic operators: the spec that names each one's inputs and the tiling it is
built at (``python/cleave/dynamic/registry.py:37-231``).  Of the reference's nine operators
All nine of the reference's operators are built: the four decode ones (paged GQA: page size 1
with 8 and 4 kv heads, page size 64; paged MLA) and the five causal prefill ones (GQA with a
token table or packed keys, 8 and 4 kv heads; paged MLA)."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..runtime.validate import Tolerance
from . import workloads as _wl
from .paging import (MLA_PAGED_PREFILL_CAUSAL, PAGED_DECODE_SLAB, PAGED_PREFILL_CAUSAL, RAGGED_PREFILL_CAUSAL, MLASpec,
                     PagingSpec)

# Paged kernels reproduce their references far more tightly than the loose default bound;
# equal_nan stays off: an empty request is defined as 0 / -inf, so a NaN is a defect.
GATHER_TOLERANCE = Tolerance(rtol=0.01, atol=0.01, equal_nan=False)


@dataclass(frozen=True)
class DynamicOperator:
    name: str
    spec: PagingSpec
    tuned_tiling: dict
    dims: tuple            # (qo_heads, kv_heads, head_dim)
    workloads: tuple
    tolerance: Tolerance = GATHER_TOLERANCE
    page_size: int = 1
    scale: float | None = None

    @property
    def is_mla(self) -> bool:
        return isinstance(self.spec, MLASpec)

    def matches(self, attention) -> bool:
        a = attention
        if self.is_mla:
            return (a.is_mla and a.kind == self.spec.kind and a.page_size == self.page_size
                    and (a.num_qo_heads, a.head_dim, a.pe_dim) == tuple(self.dims[:3]))
        return (not a.is_mla and (a.num_qo_heads, a.num_kv_heads, a.head_dim) == tuple(self.dims[:3])
                and a.page_size == self.page_size and a.kind == self.spec.kind)

    def keyed_workloads(self, *, keep: int = 0, dtype=None):
        from ..runtime.autotune import sampled, workload_key

        chosen = sampled(list(self.workloads), keep)

        def generate():
            for axes in chosen:
                inputs, expected = _wl.case(self.name, axes, self.dims, self.page_size, self.scale, dtype=dtype)
                yield workload_key(axes), inputs, expected

        return generate

    def kernel_source(self) -> str:
        """HIP source of this operator at its tuned tiling (single kernel)."""
        from ..codegen import HipCodeGen
        from .paging import DenseAttention, DenseMLA
        from .paging.apply import _mla_outputs, _mla_params, _mla_plan, _paged_outputs, _paged_params, _plan

        t = self.tuned_tiling
        if self.spec.kind in (PAGED_PREFILL_CAUSAL, RAGGED_PREFILL_CAUSAL):
            from .paging.apply import _prefill_plan

            dense = DenseAttention(16, 32, t["head_dim"], self.spec.num_kv_heads * 64, "bfloat16", "bfloat16",
                                   waves=self.spec.num_kv_heads)
            return HipCodeGen().gen(_prefill_plan(self.spec, dense, shared=True))   # the measured winner
        if self.is_mla:
            dense = DenseMLA(self.dims[0], self.dims[1], self.dims[2], "bfloat16", "bfloat16")
            params, ops = _mla_params(self.spec, dense)
            outs, out_ops = _mla_outputs(self.spec, dense)
            return HipCodeGen().gen(_mla_plan(self.spec, dense, "main", params + outs, {**ops, **out_ops}, tok=2))
        dense = DenseAttention(t["query_rows"], t["kv_tile"], t["head_dim"], t["waves"] * 64, "bfloat16", "bfloat16",
                               waves=t["waves"])
        params, ops = _paged_params(self.spec, dense)
        outs, out_ops = _paged_outputs(self.spec, dense)
        return HipCodeGen().gen(_plan(self.spec, dense, "main", params + outs, {**ops, **out_ops}))


OPERATORS = {op.name: op for op in (
    # page size 1: the row-gather layer (one table entry per token); the kv4 operator has eight
    # query rows per kv head, the kv8 one four: both fit one 16-row tile
    DynamicOperator(
        "gqa_paged_decode_h32_kv8_d128_ps1", PagingSpec(num_qo_heads=32, num_kv_heads=8),
        dict(query_rows=16, kv_tile=32, head_dim=128, waves=4), (32, 8, 128),
        _wl.WORKLOADS["gqa_paged_decode_h32_kv8_d128_ps1"], page_size=1),
    DynamicOperator(
        "gqa_paged_decode_h32_kv4_d128_ps1", PagingSpec(num_qo_heads=32, num_kv_heads=4, grid_order=("head", "batch")),
        dict(query_rows=16, kv_tile=32, head_dim=128, waves=4), (32, 4, 128),
        _wl.WORKLOADS["gqa_paged_decode_h32_kv4_d128_ps1"], page_size=1),
    DynamicOperator(
        "gqa_paged_decode_h32_kv8_d128_ps64",
        PagingSpec(num_qo_heads=32, num_kv_heads=8, kind=PAGED_DECODE_SLAB, page_size=64, grid_order=("head", "batch"),
                   pass_configs={}),
        dict(query_rows=16, kv_tile=32, head_dim=128, waves=4), (32, 8, 128),
        _wl.WORKLOADS["gqa_paged_decode_h32_kv8_d128_ps64"], page_size=64),
    # causal prefill over ragged queries: keys through a token table ...
    *(DynamicOperator(
        f"gqa_paged_prefill_causal_h32_kv{kv}_d128_ps1",
        PagingSpec(num_qo_heads=32, num_kv_heads=kv, kind=PAGED_PREFILL_CAUSAL, causal=True),
        dict(query_rows=16, kv_tile=32, head_dim=128), (32, kv, 128),
        _wl.WORKLOADS[f"gqa_paged_prefill_causal_h32_kv{kv}_d128_ps1"], page_size=1) for kv in (8, 4)),
    # ... or packed per request
    *(DynamicOperator(
        f"gqa_ragged_prefill_causal_h32_kv{kv}_d128",
        PagingSpec(num_qo_heads=32, num_kv_heads=kv, kind=RAGGED_PREFILL_CAUSAL, causal=True, rasterization=None,
                   cache_inputs=("K", "V")),
        dict(query_rows=16, kv_tile=32, head_dim=128), (32, kv, 128),
        _wl.WORKLOADS[f"gqa_ragged_prefill_causal_h32_kv{kv}_d128"], page_size=1) for kv in (8, 4)),
    # latent attention: one compressed cache (keys and values) + a rope cache, 16 heads, token table
    DynamicOperator(
        "mla_paged_decode_h16_ckv512_kpe64_ps1", MLASpec(num_qo_heads=16),
        dict(query_rows=16, kv_tile=32, n_threads=64, ckv=512, kpe=64), (16, 512, 64),
        _wl.WORKLOADS["mla_paged_decode_h16_ckv512_kpe64_ps1"], page_size=1, scale=_wl.MLA_SM_SCALE),
    DynamicOperator(
        "mla_paged_prefill_causal_h16_ckv512_kpe64_ps1",
        MLASpec(num_qo_heads=16, kind=MLA_PAGED_PREFILL_CAUSAL, causal=True, index_window_tiles=4, prefetch=False,
                rasterization=1, query_inputs=("Q_NOPE", "Q_PE"), cache_inputs=("CKV_CACHE", "KPE_CACHE"),
                index_input="KV_INDICES"),
        dict(query_rows=16, kv_tile=32, n_threads=64, ckv=512, kpe=64), (16, 512, 64),
        _wl.WORKLOADS["mla_paged_prefill_causal_h16_ckv512_kpe64_ps1"], page_size=1, scale=_wl.MLA_SM_SCALE),
)}
