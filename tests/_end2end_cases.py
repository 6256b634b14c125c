"""The reference's end-to-end case list (``tests/schedule/end2end/test_end2end.py:14-43``) in this
package's programs: name -> (program, sizes, None | "partial" | "combine").

The reference lists the halves of a split (``*_partial`` / ``*_combine``) as graphs of their own;
here they are the two stages ``split_stages`` cuts out of the unsplit program at the same
sizes.  Its attention cases subtract the constant 50 / sqrt(d) instead of a maximum; that form is
``examples.gqa_decode_shift``.
"""

import cleave_amd.lang as cl
from cleave_amd import examples as C
from cleave_amd.lower.stages import split_stages
from cleave_amd.pipeline.direct import stage_graph

SPLIT = 4
ATTN = C.gqa_decode_shift

CASES = {
    "batched_matmul_splitk_combine": (C.batched_matmul, dict(BX=2, BW=2, M=128, N=128, K=4096), "combine"),
    "batched_matmul_splitk_partial": (C.batched_matmul, dict(BX=2, BW=2, M=128, N=128, K=4096), "partial"),
    "flash_attention_sd": (ATTN, dict(HQ=1, HKV=1, SQ=4096, SKV=4096, D=64), None),
    "gqa_bhsd": (ATTN, dict(HQ=32, HKV=8, SQ=4096, SKV=4096, D=64), None),
    "lora": (C.lora, dict(M=16, N=4096, K=4096, R=16), None),
    "matmul": (C.matmul, dict(M=128, N=128, K=4096), None),
    "matmul_matmul_bhsd": (C.matmul_matmul, dict(H=32, SQ=4096, SKV=4096, D=64), None),
    "matmul_matmul_small_k": (C.matmul_matmul_2d, dict(M=4096, N=4096, K=64), None),
    "matmul_matmul_small_n": (C.matmul_matmul_2d, dict(M=4096, N=64, K=64), None),
    "matmul_rowsum_small_k": (C.matmul_rowsum, dict(M=4096, N=4096, K=64), None),
    "matmul_splitk_combine": (C.matmul, dict(M=128, N=128, K=4096), "combine"),
    "matmul_splitk_partial": (C.matmul, dict(M=128, N=128, K=4096), "partial"),
    "mha_bhsd": (ATTN, dict(HQ=32, HKV=32, SQ=4096, SKV=4096, D=64), None),
    "mha_split_combine": (ATTN, dict(HQ=32, HKV=32, SQ=4096, SKV=4096, D=64), "combine"),
    "mha_split_partial": (ATTN, dict(HQ=32, HKV=32, SQ=4096, SKV=4096, D=64), "partial"),
    "mla_decode_bhsd": (C.mla_decode, dict(B=1, H=128, D=512, PE=64, SKV=4096), None),
    "mla_prefill_bhsd": (C.mla_prefill, dict(H=128, SQ=4096, SKV=4096, DK=192, DV=128), None),
    "mqa_bhsd": (ATTN, dict(HQ=32, HKV=1, SQ=4096, SKV=4096, D=64), None),
    "qknorm": (C.qknorm, dict(HQ=64, HKV=8, SQ=4096, SKV=4096, D=128), None),
    "rmsnorm_matmul": (C.rmsnorm_matmul_plain, dict(M=4096, N=6144, K=4096), None),
    "rmsnorm_matmul_split_combine": (C.rmsnorm_matmul_plain, dict(M=1024, N=6144, K=4096), "combine"),
    "rmsnorm_matmul_split_partial": (C.rmsnorm_matmul_plain, dict(M=1024, N=6144, K=4096), "partial"),
    "rowsum": (C.rowsum, dict(M=4096, N=4096), None),
    "rowsum_div": (C.rowsum_div, dict(M=4096, N=4096), None),
    "swiglu": (C.swiglu, dict(M=4096, N=14336, K=4096), None),
}


def flat_graph(name):
    """The lowered graph of a case: the whole program, or the half of its split the name asks for."""
    program, sizes, half = CASES[name]
    graph = stage_graph(program.trace(cl.f16, **sizes))
    if half is None:
        return graph
    partial, combine = split_stages(graph, SPLIT)
    return partial if half == "partial" else combine
