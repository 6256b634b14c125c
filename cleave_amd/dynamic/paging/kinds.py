"""Names of the access layers and of the spec fields each one reads
(``python/cleave/dynamic/paging/kinds.py:3-77``)."""

PAGED_DECODE = "paged_decode"                 # one token per page-table entry
PAGED_DECODE_SLAB = "paged_decode_slab"       # page_size > 1: the table counts pages
PAGED_PREFILL_CAUSAL = "paged_prefill_causal"
RAGGED_PREFILL_CAUSAL = "ragged_prefill_causal"
KINDS = (PAGED_DECODE, PAGED_DECODE_SLAB, PAGED_PREFILL_CAUSAL, RAGGED_PREFILL_CAUSAL)
CAUSAL_KINDS = (PAGED_PREFILL_CAUSAL, RAGGED_PREFILL_CAUSAL)
PAGED_KINDS = (PAGED_DECODE, PAGED_DECODE_SLAB, PAGED_PREFILL_CAUSAL)
SLAB_KINDS = (PAGED_DECODE_SLAB,)

MLA_PAGED_DECODE = "mla_paged_decode"
MLA_PAGED_PREFILL_CAUSAL = "mla_paged_prefill_causal"
MLA_KINDS = (MLA_PAGED_DECODE, MLA_PAGED_PREFILL_CAUSAL)
SPLIT_KINDS = (PAGED_DECODE, PAGED_DECODE_SLAB, MLA_PAGED_DECODE)

# Layers this back end has a HIP template for (all of them).
BUILT_KINDS = KINDS + MLA_KINDS

# Spec fields only some layers read, each with its readers.  A spec that sets a field its layer
# does not read is refused (the field would silently do nothing); fields not listed here are
# read by every layer.
_READERS = {
    "batch_dim": (PAGED_DECODE, PAGED_DECODE_SLAB),
    "tokens_dim": CAUSAL_KINDS,
    "kv_tokens_dim": (RAGGED_PREFILL_CAUSAL,),
    "pages_dim": PAGED_KINDS,
    "index_dim": PAGED_KINDS,
    "index_input": PAGED_KINDS,
    "last_page_len_input": SLAB_KINDS,
    "query_indptr_input": CAUSAL_KINDS,
    "grid_order": (PAGED_DECODE, PAGED_DECODE_SLAB),
}
_MLA_READERS = {
    "batch_dim": (MLA_PAGED_DECODE,),
    "tokens_dim": (MLA_PAGED_PREFILL_CAUSAL,),
    "query_indptr_input": (MLA_PAGED_PREFILL_CAUSAL,),
}


def _by_layer(readers: dict, layers) -> dict:
    return {layer: {name for name, who in readers.items() if layer in who} for layer in layers}


OPTIONAL_FIELDS = tuple(_READERS)
FIELDS_READ = _by_layer(_READERS, KINDS)
MLA_OPTIONAL_FIELDS = tuple(_MLA_READERS)
MLA_FIELDS_READ = _by_layer(_MLA_READERS, MLA_KINDS)

# Partial tensors of a split-KV pair.  The reference hands over (ROWSUM, VALUE) because it
# subtracts no maximum; the exact online softmax here also carries the running maximum.
PARTIAL_MAX = "PM"
PARTIAL_ROWSUM = "PL"
PARTIAL_VALUE = "PO"
