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

OPTIONAL_FIELDS = ("batch_dim", "tokens_dim", "kv_tokens_dim", "pages_dim", "index_dim", "index_input",
                   "last_page_len_input", "query_indptr_input", "grid_order")
FIELDS_READ = {
    PAGED_DECODE: {"batch_dim", "pages_dim", "index_dim", "index_input", "grid_order"},
    PAGED_DECODE_SLAB: {"batch_dim", "pages_dim", "index_dim", "index_input", "grid_order", "last_page_len_input"},
    PAGED_PREFILL_CAUSAL: {"tokens_dim", "pages_dim", "index_dim", "index_input", "query_indptr_input"},
    RAGGED_PREFILL_CAUSAL: {"tokens_dim", "kv_tokens_dim", "query_indptr_input"},
}
MLA_OPTIONAL_FIELDS = ("batch_dim", "tokens_dim", "query_indptr_input")
MLA_FIELDS_READ = {MLA_PAGED_DECODE: {"batch_dim"}, MLA_PAGED_PREFILL_CAUSAL: {"tokens_dim", "query_indptr_input"}}

# Partial tensors of a split-KV pair.  The reference hands over (ROWSUM, VALUE) because it
# subtracts no maximum; the exact online softmax here also carries the running maximum.
PARTIAL_MAX = "PM"
PARTIAL_ROWSUM = "PL"
PARTIAL_VALUE = "PO"
