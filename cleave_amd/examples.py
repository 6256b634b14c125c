"""The five graded operators as ``@jit`` programs, with their seeded inputs.

Shapes at ``FULL`` are the benchmark configurations; ``SMALL`` are the same programs at sizes
the numpy oracle finishes in well under a second.
"""

from __future__ import annotations

import math

import torch

import cleave_amd
import cleave_amd.lang as cl


@cleave_amd.jit
def matmul(x: cl.Tensor["M", "K"], w: cl.Tensor["K", "N"]):
    return x @ w


@cleave_amd.jit
def matmul_nt(x: cl.Tensor["M", "K"], w: cl.Tensor["N", "K"]):
    """``x @ w.T`` with the weight stored (N, K), the layout of a linear layer's weight: both operands
    are contraction-minor (the reference's ``trans_B``, ``python/cleave/ir/ops/reduction.py:146-188``)."""
    return x @ w.mT


@cleave_amd.jit
def batched_matmul(x: cl.Tensor["BX", "M", "K"], w: cl.Tensor["BW", "K", "N"]):
    """``x @ w`` per batch entry; ``BX`` may be a whole multiple of ``BW`` (entries of ``w`` shared by
    groups of ``x``).  Split over K it is the reference's ``batched_matmul_splitk_partial`` /
    ``_combine`` pair, (2, 4, 128, 128, 1024) (``tests/_graphs.py:365-402``)."""
    return x @ w


@cleave_amd.jit
def rmsnorm_matmul(x: cl.Tensor["M", "K"], gamma: cl.Tensor[1, "K"], w: cl.Tensor["K", "N"]):
    return (cl.rms_norm(x, dim=-1, eps=1e-6) * gamma) @ w


@cleave_amd.jit
def rmsnorm_matmul_plain(x: cl.Tensor["M", "K"], w: cl.Tensor["K", "N"]):
    return cl.rms_norm(x, dim=-1) @ w


@cleave_amd.jit
def rmsnorm_matmul_eps(x: cl.Tensor["M", "K"], w: cl.Tensor["K", "N"]):
    return cl.rms_norm(x, dim=-1, eps=1e-2) @ w


@cleave_amd.jit
def swiglu(x: cl.Tensor["M", "K"], w_up: cl.Tensor["K", "N"], w_gate: cl.Tensor["K", "N"]):
    """``(x @ w_up) * silu(x @ w_gate)`` (the reference's ``demo/swiglu.py`` / ``tests/_graphs.py:403-436``)."""
    return (x @ w_up) * cl.silu(x @ w_gate)


@cleave_amd.jit
def lora(x: cl.Tensor["M", "K"], w: cl.Tensor["K", "N"], a: cl.Tensor["K", "R"], b: cl.Tensor["R", "N"]):
    """``x @ w + (x @ a) @ b`` (the reference's ``demo/lora.py`` / ``tests/_graphs.py:438-480``)."""
    return x @ w + (x @ a) @ b


@cleave_amd.jit
def rowsum(x: cl.Tensor["M", "N"]):
    """Row sums (the reference's ``rowsum`` case, ``tests/_graphs.py:1238-1249``)."""
    return x.sum(dim=-1, keepdim=True)


@cleave_amd.jit
def rowsum_div(x: cl.Tensor["M", "N"]):
    """Rows divided by their sums (the reference's ``rowsum_div`` case, ``tests/_graphs.py:1252-1275``)."""
    return x / x.sum(dim=-1, keepdim=True)


@cleave_amd.jit
def matmul_rowsum(x: cl.Tensor["M", "K"], w: cl.Tensor["K", "N"]):
    """Row sums of a product that is never stored (the reference's ``tests/_graphs.py:150-160``)."""
    return (x @ w).sum(dim=-1, keepdim=True)


@cleave_amd.jit
def gqa_decode_exact(q: cl.Tensor["HQ", "SQ", "D"], k: cl.Tensor["HKV", "SKV", "D"], v: cl.Tensor["HKV", "SKV", "D"]):
    return cl.softmax((q @ k.mT) / q.shape[-1] ** 0.5, dim=-1) @ v


@cleave_amd.jit
def mla_prefill(q: cl.Tensor["H", "SQ", "DK"], k: cl.Tensor["H", "SKV", "DK"], v: cl.Tensor["H", "SKV", "DV"]):
    """Attention with a key width that differs from the value width (the reference's
    ``mla_prefill_bhsd`` case, 192 / 128: ``tests/schedule/end2end/test_end2end.py:33``)."""
    return cl.softmax((q @ k.mT) / q.shape[-1] ** 0.5, dim=-1) @ v


@cleave_amd.jit
def qknorm(q: cl.Tensor["HQ", "SQ", "D"], k: cl.Tensor["HKV", "SKV", "D"], v: cl.Tensor["HKV", "SKV", "D"]):
    """Grouped-query attention over RMS-normalised queries and keys (the reference's
    ``demo/qknorm.py`` / ``tests/_graphs.py:542-640``)."""
    qn, kn = cl.rms_norm(q, dim=-1, eps=1e-6), cl.rms_norm(k, dim=-1, eps=1e-6)
    return cl.softmax((qn @ kn.mT) / q.shape[-1] ** 0.5, dim=-1) @ v


@cleave_amd.jit
def matmul_matmul(q: cl.Tensor["H", "SQ", "D"], k: cl.Tensor["H", "SKV", "D"], v: cl.Tensor["H", "SKV", "D"]):
    """``(q @ k^T) @ v`` with nothing in between (the reference's ``matmul_matmul_bhsd`` case,
    ``tests/_graphs.py:78-101``)."""
    return (q @ k.mT) @ v


@cleave_amd.jit
def matmul_matmul_2d(a: cl.Tensor["M", "K"], b: cl.Tensor["K", "N"], c: cl.Tensor["N", "K"]):
    """``(a @ b) @ c`` with the middle operand given (K, N) (the reference's ``matmul_matmul_small_k``
    (4096, 4096, 64) and ``matmul_matmul_small_n`` (4096, 64, 64) cases, ``tests/_graphs.py:65-76``)."""
    return (a @ b) @ c


@cleave_amd.jit
def gqa_decode_shift(q: cl.Tensor["HQ", "SQ", "D"], k: cl.Tensor["HKV", "SKV", "D"], v: cl.Tensor["HKV", "SKV", "D"]):
    n = q.shape[-1] ** 0.5
    return cl.softmax((q @ k.mT) / n, dim=-1, shift=-50 / n) @ v


@cleave_amd.jit
def mla_decode(q: cl.Tensor["B", "H", "D"], kv: cl.Tensor["B", "SKV", "D"], q_pe: cl.Tensor["B", "H", "PE"],
               k_pe: cl.Tensor["B", "SKV", "PE"]):
    s = (q @ kv.mT + q_pe @ k_pe.mT) * (192 ** -0.5)
    return cl.softmax(s, dim=-1) @ kv


FULL = {
    "c1": dict(M=128, N=128, K=4096),
    "c2": dict(M=16, K=4096, N=11008),
    "c3": dict(HQ=256, HKV=64, SQ=1, SKV=8192, D=128),
    "c4": dict(B=16, H=128, D=512, PE=64, SKV=4096),
    "swiglu": dict(M=4096, N=14336, K=4096),
    "matmul_rowsum": dict(M=4096, N=4096, K=64),
    "lora": dict(M=16, N=4096, K=4096, R=16),
}
SMALL = {
    "c1": dict(M=32, N=64, K=256),
    "c2": dict(M=16, K=256, N=384),
    "c3": dict(HQ=8, HKV=2, SQ=1, SKV=200, D=128),
    "c4": dict(B=2, H=16, D=512, PE=64, SKV=100),
}


def _gen(seed):
    return torch.Generator(device="cpu").manual_seed(seed)


def inputs_c1(shapes, seed=1, device="cpu"):
    g = _gen(seed)
    M, N, K = shapes["M"], shapes["N"], shapes["K"]
    x = (torch.rand(M, K, generator=g) * 2 - 1) / math.sqrt(K)
    w = (torch.rand(K, N, generator=g) * 2 - 1) / math.sqrt(K)
    return [x.to(torch.float16).to(device), w.to(torch.float16).to(device)]


def inputs_nt(shapes, seed=17, device="cpu", dtype=torch.float16):
    """x (M, K) and the weight as (N, K), both U(-1, 1) / sqrt(K)."""
    g = _gen(seed)
    M, N, K = shapes["M"], shapes["N"], shapes["K"]
    x = (torch.rand(M, K, generator=g) * 2 - 1) / math.sqrt(K)
    w = (torch.rand(N, K, generator=g) * 2 - 1) / math.sqrt(K)
    return [x.to(dtype).to(device), w.to(dtype).to(device)]


def inputs_nt_bf16(shapes, seed=18, device="cpu"):
    return inputs_nt(shapes, seed=seed, device=device, dtype=torch.bfloat16)


def inputs_batched(shapes, seed=14, device="cpu"):
    g = _gen(seed)
    bx, bw, M, N, K = (shapes[k] for k in ("BX", "BW", "M", "N", "K"))
    x = (torch.rand(bx, M, K, generator=g) * 2 - 1) / math.sqrt(K)
    w = (torch.rand(bw, K, N, generator=g) * 2 - 1) / math.sqrt(K)
    return [x.to(torch.float16).to(device), w.to(torch.float16).to(device)]


def inputs_plain_norm(shapes, seed=15, device="cpu"):
    g = _gen(seed)
    M, N, K = shapes["M"], shapes["N"], shapes["K"]
    x = torch.randn(M, K, generator=g)
    w = torch.randn(K, N, generator=g) / math.sqrt(K)
    return [x.to(torch.float16).to(device), w.to(torch.float16).to(device)]


def inputs_chain2d(shapes, seed=16, device="cpu"):
    """a (M, K) scaled so that sums of thousands of products stay inside f16, b (K, N), c (N, K)."""
    g = _gen(seed)
    M, N, K = shapes["M"], shapes["N"], shapes["K"]
    a, b, c = torch.randn(M, K, generator=g) / 8, torch.randn(K, N, generator=g), torch.randn(N, K, generator=g)
    return [t.to(torch.float16).to(device) for t in (a, b, c)]


def inputs_swiglu(shapes, seed=6, device="cpu"):
    g = _gen(seed)
    M, N, K = shapes["M"], shapes["N"], shapes["K"]
    x = torch.randn(M, K, generator=g)
    ws = [torch.randn(K, N, generator=g) / math.sqrt(K) for _ in range(2)]
    return [t.to(torch.float16).to(device) for t in (x, *ws)]


def inputs_rows(shapes, seed=12, device="cpu"):
    g = _gen(seed)
    return [(torch.rand(shapes["M"], shapes["N"], generator=g) + 0.25).to(torch.float16).to(device)]


def inputs_lora(shapes, seed=9, device="cpu"):
    g = _gen(seed)
    M, N, K, R = shapes["M"], shapes["N"], shapes["K"], shapes["R"]
    x = torch.randn(M, K, generator=g)
    w = torch.randn(K, N, generator=g) / math.sqrt(K)
    a = torch.randn(K, R, generator=g) / math.sqrt(K)
    b = torch.randn(R, N, generator=g) / math.sqrt(R)
    return [t.to(torch.float16).to(device) for t in (x, w, a, b)]


def inputs_c2(shapes, seed=2, device="cpu"):
    g = _gen(seed)
    M, N, K = shapes["M"], shapes["N"], shapes["K"]
    x = torch.randn(M, K, generator=g)
    gamma = 1 + 0.1 * torch.randn(1, K, generator=g)
    w = torch.randn(K, N, generator=g) / math.sqrt(K)
    return [t.to(torch.float16).to(device) for t in (x, gamma, w)]


def inputs_c3(shapes, seed=3, device="cpu"):
    g = _gen(seed)
    s = shapes
    q = torch.randn(s["HQ"], s["SQ"], s["D"], generator=g)
    k = torch.randn(s["HKV"], s["SKV"], s["D"], generator=g)
    v = torch.randn(s["HKV"], s["SKV"], s["D"], generator=g)
    return [t.to(torch.float16).to(device) for t in (q, k, v)]


def inputs_mla_prefill(shapes, seed=8, device="cpu"):
    g = _gen(seed)
    s = shapes
    q = torch.randn(s["H"], s["SQ"], s["DK"], generator=g)
    k = torch.randn(s["H"], s["SKV"], s["DK"], generator=g)
    v = torch.randn(s["H"], s["SKV"], s["DV"], generator=g)
    return [t.to(torch.float16).to(device) for t in (q, k, v)]


def inputs_c4(shapes, seed=4, device="cpu"):
    g = _gen(seed)
    s = shapes
    q = 0.5 * torch.randn(s["B"], s["H"], s["D"], generator=g)
    kv = 0.5 * torch.randn(s["B"], s["SKV"], s["D"], generator=g)
    q_pe = 0.5 * torch.randn(s["B"], s["H"], s["PE"], generator=g)
    k_pe = 0.5 * torch.randn(s["B"], s["SKV"], s["PE"], generator=g)
    return [t.to(torch.bfloat16).to(device) for t in (q, kv, q_pe, k_pe)]


CASES = {
    "c1": (matmul, cl.f16, inputs_c1),
    "c2": (rmsnorm_matmul, cl.f16, inputs_c2),
    "c3": (gqa_decode_exact, cl.f16, inputs_c3),
    "c4": (mla_decode, cl.bf16, inputs_c4),
}


def paged_workload(lens, page_size=64, num_pages=None, hq=32, hkv=8, d=128, seed=5, dtype=torch.float16,
                   device="cpu", pool_scale=1.0):
    """C5-style paged decode arguments: q, k_cache, v_cache, kv_indptr, kv_indices,
    kv_last_page_len, sm_scale.  The block table is a seeded random permutation of the pool."""
    g = _gen(seed)
    pages = [-(-n // page_size) for n in lens]
    total = sum(pages)
    num_pages = num_pages or max(total, 1)
    kv_indices = torch.randperm(num_pages, generator=g)[:total].to(torch.int32)
    indptr = torch.tensor([0] + list(torch.tensor(pages).cumsum(0).tolist()), dtype=torch.int32)
    last = torch.tensor([n - (p - 1) * page_size if p else 0 for n, p in zip(lens, pages)], dtype=torch.int32)
    q = torch.randn(len(lens), hq, d, generator=g).to(dtype)
    k_cache = (torch.randn(num_pages, page_size, hkv, d, generator=g) * pool_scale).to(dtype)
    v_cache = (torch.randn(num_pages, page_size, hkv, d, generator=g) * pool_scale).to(dtype)
    args = [q, k_cache, v_cache, indptr, kv_indices, last]
    return [a.to(device) for a in args] + [float(d) ** -0.5]


_batch, _num_pages, _n_idx = cl.dims("batch num_pages n_idx", dynamic=True)
_kv_len = cl.Dim("kv_len", dynamic=True, hint=4096)


def paged_decode_op(hq=32, hkv=8, d=128, page=64, dtype=cl.f16, name=None):
    """The paged GQA decode operator as a ``@jit`` program (the reference's registry form:
    with a last-page-length input only when pages hold more than one token)."""
    name = name or f"gqa_paged_decode_h{hq}_kv{hkv}_d{d}_ps{page}"

    def body(q, k_cache, v_cache, pages):
        k, v = cl.paged_gather(k_cache, pages), cl.paged_gather(v_cache, pages)
        qg = q.view(_batch, hkv, hq // hkv, d)
        return qg, k, v

    if page > 1:
        def op(q, k_cache, v_cache, kv_indptr, kv_indices, kv_last_page_len, sm_scale):
            pages = cl.PageTable(kv_indptr, kv_indices, last_page_len=kv_last_page_len, length=_kv_len)
            qg, k, v = body(q, k_cache, v_cache, pages)
            p, lse = cl.softmax((qg @ k.mT) * sm_scale, dim=-1, return_lse=True)
            return (p @ v).view(_batch, hq, d), lse.view(_batch, hq)
    else:
        def op(q, k_cache, v_cache, kv_indptr, kv_indices, sm_scale):
            pages = cl.PageTable(kv_indptr, kv_indices, length=_kv_len)
            qg, k, v = body(q, k_cache, v_cache, pages)
            p, lse = cl.softmax((qg @ k.mT) * sm_scale, dim=-1, return_lse=True)
            return (p @ v).view(_batch, hq, d), lse.view(_batch, hq)
    # the annotations are built here rather than written on the signature: this module defers
    # annotation evaluation, and the extents are arguments of this factory
    ann = {"q": cl.Tensor[_batch, hq, d], "k_cache": cl.Tensor[_num_pages, page, hkv, d],
           "v_cache": cl.Tensor[_num_pages, page, hkv, d], "kv_indptr": cl.Tensor[_batch + 1, cl.i32],
           "kv_indices": cl.Tensor[_n_idx, cl.i32], "sm_scale": cl.Scalar[cl.f32]}
    if page > 1:
        ann["kv_last_page_len"] = cl.Tensor[_batch, cl.i32] | None
    op.__annotations__ = ann
    return cleave_amd.jit(name=name, dtype=dtype)(op)


def mla_paged_decode_op(heads=16, ckv=512, kpe=64, dtype=cl.bf16, name=None):
    """The paged MLA decode operator as a ``@jit`` program (the reference's registry form,
    ``demo/dynamic/mla_paged_decode.py``): one compressed cache that is both keys and values, a
    rope cache adding a second score term, a token table (page size 1)."""
    name = name or f"mla_paged_decode_h{heads}_ckv{ckv}_kpe{kpe}_ps1"

    def op(qn, qp, ckv_cache, kpe_cache, kv_indptr, kvi, sm_scale):
        pages = cl.PageTable(kv_indptr, kvi, length=_kv_len)
        c, r = cl.paged_gather(ckv_cache, pages), cl.paged_gather(kpe_cache, pages)
        p, lse = cl.softmax((qn @ c.mT + qp @ r.mT) * sm_scale, dim=-1, return_lse=True)
        return p @ c, lse

    op.__annotations__ = {"qn": cl.Tensor[_batch, heads, ckv], "qp": cl.Tensor[_batch, heads, kpe],
                          "ckv_cache": cl.Tensor[_num_pages, 1, ckv], "kpe_cache": cl.Tensor[_num_pages, 1, kpe],
                          "kv_indptr": cl.Tensor[_batch + 1, cl.i32], "kvi": cl.Tensor[_n_idx, cl.i32],
                          "sm_scale": cl.Scalar[cl.f32]}
    return cleave_amd.jit(name=name, dtype=dtype)(op)


_total_q, _total_kv = cl.dims("total_q total_kv", dynamic=True)
_q_len = cl.Dim("q_len", dynamic=True)


def prefill_op(hq=32, hkv=8, d=128, ragged=False, dtype=cl.bf16, name=None):
    """The causal prefill operators as ``@jit`` programs (the reference's registry forms,
    ``demo/dynamic/gqa_paged_prefill.py`` / ``gqa_ragged_prefill.py``): ragged query rows per
    request; keys through a token table, or packed per request."""
    g = hq // hkv
    if ragged:
        name = name or f"gqa_ragged_prefill_causal_h{hq}_kv{hkv}_d{d}"

        def op(q, k, v, qo_indptr, kv_indptr, sm_scale):
            rows = cl.PageTable(qo_indptr, length=_q_len)
            keys = cl.PageTable(kv_indptr, length=_kv_len)
            qr = cl.paged_gather(q, rows).view(_batch, hkv, g, _q_len, d)
            kr = cl.paged_gather(k, keys).view(_batch, hkv, 1, _kv_len, d)
            vr = cl.paged_gather(v, keys).view(_batch, hkv, 1, _kv_len, d)
            p, lse = cl.softmax((qr @ kr.mT) * sm_scale, dim=-1, causal=True, return_lse=True)
            return (p @ vr).view(_total_q, hq, d), lse.view(_total_q, hq)

        op.__annotations__ = {"q": cl.Tensor[_total_q, hq, d], "k": cl.Tensor[_total_kv, hkv, d],
                              "v": cl.Tensor[_total_kv, hkv, d], "qo_indptr": cl.Tensor[_batch + 1, cl.i32],
                              "kv_indptr": cl.Tensor[_batch + 1, cl.i32], "sm_scale": cl.Scalar[cl.f32]}
    else:
        name = name or f"gqa_paged_prefill_causal_h{hq}_kv{hkv}_d{d}_ps1"

        def op(q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, sm_scale):
            rows = cl.PageTable(qo_indptr, length=_q_len)
            pages = cl.PageTable(kv_indptr, kv_indices, length=_kv_len)
            qr = cl.paged_gather(q, rows).view(_batch, hkv, g, _q_len, d)
            k = cl.paged_gather(k_cache, pages).view(_batch, hkv, 1, _kv_len, d)
            v = cl.paged_gather(v_cache, pages).view(_batch, hkv, 1, _kv_len, d)
            p, lse = cl.softmax((qr @ k.mT) * sm_scale, dim=-1, causal=True, return_lse=True)
            return (p @ v).view(_total_q, hq, d), lse.view(_total_q, hq)

        op.__annotations__ = {"q": cl.Tensor[_total_q, hq, d], "k_cache": cl.Tensor[_num_pages, 1, hkv, d],
                              "v_cache": cl.Tensor[_num_pages, 1, hkv, d], "qo_indptr": cl.Tensor[_batch + 1, cl.i32],
                              "kv_indptr": cl.Tensor[_batch + 1, cl.i32], "kv_indices": cl.Tensor[_n_idx, cl.i32],
                              "sm_scale": cl.Scalar[cl.f32]}
    return cleave_amd.jit(name=name, dtype=dtype)(op)


def mla_paged_prefill_op(heads=16, ckv=512, kpe=64, dtype=cl.bf16, name=None):
    """The paged MLA causal prefill operator as a ``@jit`` program (the reference's registry form,
    ``demo/dynamic/mla_paged_prefill.py``)."""
    name = name or f"mla_paged_prefill_causal_h{heads}_ckv{ckv}_kpe{kpe}_ps1"

    def op(q_nope, q_pe, ckv_cache, kpe_cache, qo_indptr, kv_indptr, kv_indices, sm_scale):
        rows = cl.PageTable(qo_indptr, length=_q_len)
        pages = cl.PageTable(kv_indptr, kv_indices, length=_kv_len)
        qn, qp = cl.paged_gather(q_nope, rows), cl.paged_gather(q_pe, rows)     # (batch, heads, q_len, width)
        c = cl.paged_gather(ckv_cache, pages).view(_batch, 1, _kv_len, ckv)
        r = cl.paged_gather(kpe_cache, pages).view(_batch, 1, _kv_len, kpe)
        p, lse = cl.softmax((qn @ c.mT + qp @ r.mT) * sm_scale, dim=-1, causal=True, return_lse=True)
        return (p @ c).view(_total_q, heads, ckv), lse.view(_total_q, heads)

    op.__annotations__ = {"q_nope": cl.Tensor[_total_q, heads, ckv], "q_pe": cl.Tensor[_total_q, heads, kpe],
                          "ckv_cache": cl.Tensor[_num_pages, 1, ckv], "kpe_cache": cl.Tensor[_num_pages, 1, kpe],
                          "qo_indptr": cl.Tensor[_batch + 1, cl.i32], "kv_indptr": cl.Tensor[_batch + 1, cl.i32],
                          "kv_indices": cl.Tensor[_n_idx, cl.i32], "sm_scale": cl.Scalar[cl.f32]}
    return cleave_amd.jit(name=name, dtype=dtype)(op)
