"""Paged access layers over the dense decode-attention and MLA decode templates."""

from .apply import (DenseAttention, DenseMLA, apply_paging, apply_paging_split, build_split_decode, can_page,
                    paging_accept, read_dense, read_dense_attention, read_dense_combine, read_dense_mla,
                    read_dense_partial)
from .errors import InvalidSpec, NotDenseAttention, PagingRefusal, UnsupportedTiling
from .kinds import (BUILT_KINDS, CAUSAL_KINDS, KINDS, MLA_KINDS, MLA_PAGED_DECODE, MLA_PAGED_PREFILL_CAUSAL,
                    PAGED_DECODE, PAGED_DECODE_SLAB, PAGED_KINDS, PAGED_PREFILL_CAUSAL, PARTIAL_MAX, PARTIAL_ROWSUM,
                    PARTIAL_VALUE, RAGGED_PREFILL_CAUSAL, SLAB_KINDS, SPLIT_KINDS)
from .specs import CombineTiling, MLASpec, PagingSpec

DENOM_FLOOR = 1e-30           # floor of the normalising division: an empty request gives 0, not NaN
LOG2E = 1.4426950408889634
