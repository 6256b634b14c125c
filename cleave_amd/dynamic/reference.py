"""Inputs and torch references of the paged attention operators, used to validate candidates.

Restates ``python/cleave/dynamic/reference.py:23-200`` for the layers this back end builds,
with two differences: the element dtype is a parameter (the reference hard-codes bf16 at
``:19,136-140``) and so is the device (default "cuda").  Conventions kept: page tables are a
seeded random permutation of the pool so the gather is genuinely scattered (``:44-49``); a
request with no keys yields 0 in the output and -inf in the base-2 lse (``:71-82``); logits
are evaluated in fp32, in query chunks so they stay bounded (``:62-105``).
"""

from __future__ import annotations

import math

SEED = 0
NEG_INF = float("-inf")
CHUNK_ELEMS = 1 << 27   # most fp32 logits alive at once


def _torch():
    import torch

    return torch


def _indptr(lengths) -> list:
    out = [0]
    for n in lengths:
        out.append(out[-1] + int(n))
    return out


def _i32(values, device):
    torch = _torch()
    return torch.tensor(list(values), device=device, dtype=torch.int32)


def _generator(device, seed=SEED):
    torch = _torch()
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)
    return gen


def _page_table(num_pages, count, device, seed=SEED):
    torch = _torch()
    perm = torch.randperm(num_pages, device=device, generator=_generator(device, seed))
    return perm[:count].to(torch.int32)


def _pad_indices(kv_indices, n_idx):
    torch = _torch()
    short = n_idx - kv_indices.numel()
    assert short >= 0, (kv_indices.numel(), n_idx)
    if short == 0:
        return kv_indices
    return torch.cat([kv_indices, torch.zeros(short, device=kv_indices.device, dtype=torch.int32)])


def _finish(logits):
    """Softmax weights and base-2 lse of a (n_q, heads, n_kv) block; fully masked rows get zero
    weights and -inf instead of NaN."""
    torch = _torch()
    lse = torch.logsumexp(logits, dim=-1) / math.log(2.0)
    weights = torch.softmax(logits, dim=-1)
    dead = torch.isneginf(lse)
    if dead.any():
        weights = weights.masked_fill(dead[..., None], 0.0)
    return weights, lse


def _attend(q, k, v, scale, mask=None):
    """One request: ``q`` (n_q, heads, d), ``k``/``v`` (n_kv, heads, d) -> out fp32, lse."""
    torch = _torch()
    n_q, heads, _ = q.shape
    kf, vf = k.float(), v.float()
    step = max(1, min(n_q, CHUNK_ELEMS // max(1, heads * k.shape[0])))
    outs, lses = [], []
    for lo in range(0, n_q, step):
        hi = min(lo + step, n_q)
        logits = torch.einsum("qhd,khd->qhk", q[lo:hi].float(), kf) * scale
        if mask is not None:
            logits = logits.masked_fill(~mask[lo:hi, None, :], NEG_INF)
        w, lse = _finish(logits)
        outs.append(torch.einsum("qhk,khd->qhd", w, vf))
        lses.append(lse)
    return torch.cat(outs), torch.cat(lses)


def paged_tokens(kv_indices, base, kv_len, page_size):
    """``(page_of, slot_of)`` for the ``kv_len`` tokens of the request whose table slice starts at
    ``base``: pages in table order, each page's slots in order, clipped to the length."""
    torch = _torch()
    n_pages = -(-kv_len // page_size)
    pages = kv_indices[base:base + n_pages].long()
    if page_size == 1:
        return pages, torch.zeros_like(pages)
    slot = torch.arange(page_size, device=kv_indices.device)
    page_of = pages[:, None].expand(-1, page_size).reshape(-1)[:kv_len]
    slot_of = slot[None, :].expand(pages.numel(), -1).reshape(-1)[:kv_len]
    return page_of, slot_of


def gqa_paged_decode_inputs(dims, kv_lens, page_size=1, scale=None, dtype=None, device="cuda", seed=SEED):
    """The operator's arguments in declaration order: q, k_cache, v_cache, kv_indptr, kv_indices,
    [kv_last_page_len], sm_scale.  ``dims`` = (batch, qo_heads, kv_heads, head_dim, num_pages, n_idx)."""
    torch = _torch()
    dtype = dtype or torch.bfloat16
    batch, hq, hkv, d, num_pages, n_idx = dims[:6]
    gen = _generator(device, seed)
    pages_per_req = [-(-int(n) // page_size) for n in kv_lens]
    kv_indices = _pad_indices(_page_table(num_pages, sum(pages_per_req), device, seed), n_idx)

    def randn(*shape):
        return torch.randn(*shape, device=device, dtype=dtype, generator=gen)

    args = [randn(batch, hq, d), randn(num_pages, page_size, hkv, d), randn(num_pages, page_size, hkv, d),
            _i32(_indptr(pages_per_req), device), kv_indices]
    if page_size != 1:
        args.append(_i32([n - (p - 1) * page_size if p else 0 for n, p in zip(kv_lens, pages_per_req)], device))
    args.append(float(d) ** -0.5 if scale is None else float(scale))
    return args


def gqa_paged_decode_reference(dims, kv_lens, page_size=1, dtype=None):
    torch = _torch()
    dtype = dtype or torch.bfloat16
    batch, hq, hkv, d = dims[:4]
    group = hq // hkv

    def reference(q, k_cache, v_cache, kv_indptr, kv_indices, *rest):
        sm_scale = rest[-1]
        out = torch.zeros(batch, hq, d, device=q.device, dtype=dtype)
        lse = torch.full((batch, hq), NEG_INF, device=q.device, dtype=torch.float32)
        starts = kv_indptr.tolist()
        for b, kv_len in enumerate(kv_lens):
            if kv_len <= 0:
                continue
            page_of, slot_of = paged_tokens(kv_indices, int(starts[b]), int(kv_len), page_size)
            kk = k_cache[page_of, slot_of].repeat_interleave(group, dim=1)
            vv = v_cache[page_of, slot_of].repeat_interleave(group, dim=1)
            o, l = _attend(q[b:b + 1], kk, vv, sm_scale)
            out[b] = o[0].to(dtype)
            lse[b] = l[0]
        return [out, lse]

    return reference


# ----------------------------------------------------------------------------- MLA paged decode
def _mla_attend_rows(qn, qp, kc, kp, scale, keep=None):
    """MLA over a block of query rows (``python/cleave/dynamic/reference.py:108-126``): ``qn``
    (n_q, heads, ckv), ``qp`` (n_q, heads, kpe), ``kc`` (n_kv, ckv) both keys and values, ``kp``
    (n_kv, kpe) -> out fp32 (n_q, heads, ckv), base-2 lse (n_q, heads)."""
    torch = _torch()
    n_q, heads, _ = qn.shape
    kcf, kpf = kc.float(), kp.float()
    step = max(1, min(n_q, CHUNK_ELEMS // max(1, heads * kc.shape[0])))
    outs, lses = [], []
    for lo in range(0, n_q, step):
        hi = min(lo + step, n_q)
        logits = (torch.einsum("qhd,kd->qhk", qn[lo:hi].float(), kcf)
                  + torch.einsum("qhd,kd->qhk", qp[lo:hi].float(), kpf)) * scale
        if keep is not None:
            logits = logits.masked_fill(~keep[lo:hi, None, :], NEG_INF)
        w, lse = _finish(logits)
        outs.append(torch.einsum("qhk,kd->qhd", w, kcf))
        lses.append(lse)
    return torch.cat(outs), torch.cat(lses)


def mla_paged_decode_inputs(dims, kv_lens, scale=None, dtype=None, device="cuda", seed=SEED):
    """The operator's arguments in declaration order (``python/cleave/dynamic/reference.py:282-295``):
    q_nope, q_pe, ckv_cache, kpe_cache, kv_indptr, kv_indices, sm_scale.
    ``dims`` = (batch, qo_heads, ckv, kpe, num_pages, n_idx)."""
    torch = _torch()
    dtype = dtype or torch.bfloat16
    batch, heads, ckv, kpe, num_pages, n_idx = dims[:6]
    gen = _generator(device, seed)
    kv_indices = _pad_indices(_page_table(num_pages, sum(int(n) for n in kv_lens), device, seed), n_idx)

    def randn(*shape):
        return torch.randn(*shape, device=device, dtype=dtype, generator=gen)

    return [randn(batch, heads, ckv), randn(batch, heads, kpe), randn(num_pages, 1, ckv), randn(num_pages, 1, kpe),
            _i32(_indptr(kv_lens), device), kv_indices, float(ckv + kpe) ** -0.5 if scale is None else float(scale)]


def mla_paged_decode_reference(dims, kv_lens, dtype=None):
    """``python/cleave/dynamic/reference.py:297-321``: per request, the rows its table slice names
    (page size 1) attended by its one query row per head; empty requests stay 0 / -inf."""
    torch = _torch()
    dtype = dtype or torch.bfloat16
    batch, heads, ckv = dims[:3]

    def reference(q_nope, q_pe, ckv_cache, kpe_cache, kv_indptr, kv_indices, sm_scale):
        out = torch.zeros(batch, heads, ckv, device=q_nope.device, dtype=dtype)
        lse = torch.full((batch, heads), NEG_INF, device=q_nope.device, dtype=torch.float32)
        starts = kv_indptr.tolist()
        for b, kv_len in enumerate(kv_lens):
            if kv_len <= 0:
                continue
            base = int(starts[b])
            pages = kv_indices[base:base + int(kv_len)].long()
            o, l = _mla_attend_rows(q_nope[b:b + 1], q_pe[b:b + 1], ckv_cache[pages, 0], kpe_cache[pages, 0], sm_scale)
            out[b] = o[0].to(dtype)
            lse[b] = l[0]
        return [out, lse]

    return reference


# ----------------------------------------------------------------------------- causal prefill
def causal_keep(q_len, kv_len, device):
    """End-aligned causal mask (``python/cleave/dynamic/reference.py:129-133``): keep
    ``kv_pos <= kv_len - q_len + q_pos``; (q_len, kv_len) bool."""
    torch = _torch()
    q_pos = torch.arange(q_len, device=device)[:, None]
    kv_pos = torch.arange(kv_len, device=device)[None, :]
    return kv_pos <= (kv_len - q_len) + q_pos


def gqa_paged_prefill_inputs(dims, q_lens, kv_lens, scale=None, dtype=None, device="cuda", seed=SEED):
    """q, k_cache, v_cache, qo_indptr, kv_indptr, kv_indices, sm_scale
    (``python/cleave/dynamic/reference.py:204-219``); ``dims`` = (qo_heads, kv_heads, head_dim,
    num_pages, n_idx, total_q)."""
    torch = _torch()
    dtype = dtype or torch.bfloat16
    hq, hkv, d, num_pages, n_idx, total_q = dims[:6]
    gen = _generator(device, seed)
    kv_indptr = _indptr(kv_lens)
    kv_indices = _pad_indices(_page_table(num_pages, kv_indptr[-1], device, seed), n_idx)

    def randn(*shape):
        return torch.randn(*shape, device=device, dtype=dtype, generator=gen)

    return [randn(total_q, hq, d), randn(num_pages, 1, hkv, d), randn(num_pages, 1, hkv, d),
            _i32(_indptr(q_lens), device), _i32(kv_indptr, device), kv_indices,
            float(d) ** -0.5 if scale is None else float(scale)]


def gqa_ragged_prefill_inputs(dims, q_lens, kv_lens, scale=None, dtype=None, device="cuda", seed=SEED):
    """q, k, v, qo_indptr, kv_indptr, sm_scale (``python/cleave/dynamic/reference.py:245-255``);
    ``dims`` = (qo_heads, kv_heads, head_dim, total_q, total_kv)."""
    torch = _torch()
    dtype = dtype or torch.bfloat16
    hq, hkv, d, total_q, total_kv = dims[:5]
    gen = _generator(device, seed)

    def randn(*shape):
        return torch.randn(*shape, device=device, dtype=dtype, generator=gen)

    return [randn(total_q, hq, d), randn(total_kv, hkv, d), randn(total_kv, hkv, d), _i32(_indptr(q_lens), device),
            _i32(_indptr(kv_lens), device), float(d) ** -0.5 if scale is None else float(scale)]


def _prefill_reference(hq, hkv, d, total_q, q_lens, kv_lens, dtype, rows_of):
    """Shared body of the two prefill references (``reference.py:221-242,258-278``): per request
    with both lengths positive, its query rows attend its keys under the end-aligned causal mask;
    everything else stays 0 / -inf.  ``rows_of(r, kv_len, tensors)`` -> (K rows, V rows)."""
    torch = _torch()
    group = hq // hkv

    def reference(q, *rest):
        sm_scale = rest[-1]
        qo_indptr = rest[2].tolist()
        out = torch.zeros(total_q, hq, d, device=q.device, dtype=dtype)
        lse = torch.full((total_q, hq), NEG_INF, device=q.device, dtype=torch.float32)
        for r, (q_len, kv_len) in enumerate(zip(q_lens, kv_lens)):
            if q_len <= 0 or kv_len <= 0:
                continue
            qs, qe = int(qo_indptr[r]), int(qo_indptr[r + 1])
            kk, vv = rows_of(r, int(kv_len), rest)
            o, l = _attend(q[qs:qe], kk.repeat_interleave(group, dim=1), vv.repeat_interleave(group, dim=1), sm_scale,
                           causal_keep(int(q_len), int(kv_len), q.device))
            out[qs:qe] = o.to(dtype)
            lse[qs:qe] = l
        return [out, lse]

    return reference


def gqa_paged_prefill_reference(dims, q_lens, kv_lens, dtype=None):
    torch = _torch()
    hq, hkv, d, _pages, _n_idx, total_q = dims[:6]

    def rows_of(r, kv_len, rest):
        k_cache, v_cache, _qo, kv_indptr, kv_indices = rest[:5]
        base = int(kv_indptr[r])
        pages = kv_indices[base:base + kv_len].long()
        return k_cache[pages, 0], v_cache[pages, 0]

    return _prefill_reference(hq, hkv, d, total_q, q_lens, kv_lens, dtype or torch.bfloat16, rows_of)


def gqa_ragged_prefill_reference(dims, q_lens, kv_lens, dtype=None):
    torch = _torch()
    hq, hkv, d, total_q, _total_kv = dims[:5]

    def rows_of(r, kv_len, rest):
        k, v, _qo, kv_indptr = rest[:4]
        ks = int(kv_indptr[r])
        return k[ks:ks + kv_len], v[ks:ks + kv_len]

    return _prefill_reference(hq, hkv, d, total_q, q_lens, kv_lens, dtype or torch.bfloat16, rows_of)


# ----------------------------------------------------------------------------- MLA paged prefill
def mla_paged_prefill_inputs(dims, q_lens, kv_lens, scale=None, dtype=None, device="cuda", seed=SEED):
    """q_nope, q_pe, ckv_cache, kpe_cache, qo_indptr, kv_indptr, kv_indices, sm_scale
    (``python/cleave/dynamic/reference.py:324-339``); ``dims`` = (qo_heads, ckv, kpe, num_pages,
    n_idx, total_q)."""
    torch = _torch()
    dtype = dtype or torch.bfloat16
    heads, ckv, kpe, num_pages, n_idx, total_q = dims[:6]
    gen = _generator(device, seed)
    kv_indptr = _indptr(kv_lens)
    kv_indices = _pad_indices(_page_table(num_pages, kv_indptr[-1], device, seed), n_idx)

    def randn(*shape):
        return torch.randn(*shape, device=device, dtype=dtype, generator=gen)

    return [randn(total_q, heads, ckv), randn(total_q, heads, kpe), randn(num_pages, 1, ckv), randn(num_pages, 1, kpe),
            _i32(_indptr(q_lens), device), _i32(kv_indptr, device), kv_indices,
            float(ckv + kpe) ** -0.5 if scale is None else float(scale)]


def mla_paged_prefill_reference(dims, q_lens, kv_lens, dtype=None):
    """``python/cleave/dynamic/reference.py:341-370``: per request with both lengths positive, its
    query rows attend the rows its table slice names under the end-aligned causal mask."""
    torch = _torch()
    dtype = dtype or torch.bfloat16
    heads, ckv, _kpe, _pages, _n_idx, total_q = dims[:6]

    def reference(q_nope, q_pe, ckv_cache, kpe_cache, qo_indptr, kv_indptr, kv_indices, sm_scale):
        out = torch.zeros(total_q, heads, ckv, device=q_nope.device, dtype=dtype)
        lse = torch.full((total_q, heads), NEG_INF, device=q_nope.device, dtype=torch.float32)
        qo, kvp = qo_indptr.tolist(), kv_indptr.tolist()
        for r, (q_len, kv_len) in enumerate(zip(q_lens, kv_lens)):
            if q_len <= 0 or kv_len <= 0:
                continue
            qs, qe = int(qo[r]), int(qo[r + 1])
            pages = kv_indices[int(kvp[r]):int(kvp[r]) + int(kv_len)].long()
            o, l = _mla_attend_rows(q_nope[qs:qe], q_pe[qs:qe], ckv_cache[pages, 0], kpe_cache[pages, 0], sm_scale,
                                    causal_keep(int(q_len), int(kv_len), q_nope.device))
            out[qs:qe] = o.to(dtype)
            lse[qs:qe] = l
        return [out, lse]

    return reference
