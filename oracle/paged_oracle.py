"""numpy restatement of the paged GQA decode reference (reference
``python/cleave/dynamic/reference.py:143-200``) and of the integer arithmetic of the slab
access layer.  TEST INFRASTRUCTURE: see the package docstring.

  * ``paged_tokens``     ``_paged_tokens`` (``reference.py:143-152``): the cache rows a request's
                         pages cover, in order, clipped to its length;
  * ``gather``           ``k_cache[page_of, slot_of]`` (``:192-193``) as a pure index copy; the
                         bit-exactness oracle of the block-table gather;
  * ``decode``           ``gqa_paged_decode_reference`` (``:180-200``) with ``_attend`` /
                         ``_finish`` (``:62-105``): fp32 logits ``q k^T * scale``, softmax, base-2
                         lse, ``repeat_interleave`` of kv heads over the group, 0 / -inf for an
                         empty request;
  * ``valid_len``        the slab layer's length formula (``paging/builders/slab.py:138-142``):
                         ``min(max(n_pages-1, 0)*P + max(last, 0), n_pages*P)``;
  * ``split_ranges``     ``tile0`` / ``my_trip`` (``paging/stages.py:331-347``): tiles dealt
                         ``ceil(n_tiles / split)`` per split, a trailing split may get none;
  * ``mla_attend`` / ``mla_decode``   ``_mla_attend_rows`` (``reference.py:108-126``) and
                         ``mla_paged_decode_reference`` (``:297-321``): logits
                         ``(q_nope c^T + q_pe r^T) * scale`` over the rows a request's table slice
                         names (page size 1), softmax, values = the same latent rows ``c``.
                         Pins (tests/test_oracle.py): equals ``attend`` on the concatenated
                         operands (the sum of two products is one product over joined features),
                         float64 brute force, page-permutation invariance, 0 / -inf for an empty
                         request;
  * ``causal_keep`` / ``prefill``   ``_causal_keep`` (``reference.py:129-133``: keep
                         ``kv_pos <= kv_len - q_len + q_pos``) and the two causal prefill
                         references (``:221-242`` token table, ``:258-278`` packed keys): ragged
                         query rows per request, fully masked rows 0 / -inf.  Pins
                         (tests/test_oracle.py): a request with one query row equals ``decode``
                         of the same keys; row i equals ``attend`` over the first
                         ``kv_len - q_len + i + 1`` keys (the mask as a prefix length); rows with
                         ``kv_len - q_len + i < 0`` are 0 / -inf; token-table and packed forms
                         agree on the same rows;
  * ``mla_prefill``      ``mla_paged_prefill_reference`` (``reference.py:341-370``): the MLA scores
                         and latent values of ``mla_attend`` under ``causal_keep``.  Pin: equals
                         ``prefill`` on the joined features with the latent part as values.
"""

from __future__ import annotations

import math

import numpy as np

from .program_oracle import round_to_dtype, to_f32


def paged_tokens(kv_indices: np.ndarray, base: int, kv_len: int, page_size: int):
    n_pages = -(-kv_len // page_size)
    pages = np.asarray(kv_indices[base:base + n_pages], dtype=np.int64)
    if page_size == 1:
        return pages, np.zeros_like(pages)
    page_of = np.repeat(pages, page_size)[:kv_len]
    slot_of = np.tile(np.arange(page_size, dtype=np.int64), len(pages))[:kv_len]
    return page_of, slot_of


def gather(cache: np.ndarray, kv_indices, base: int, kv_len: int, page_size: int) -> np.ndarray:
    """``cache[page_of, slot_of]``: (kv_len, kv_heads, d), bits untouched."""
    page_of, slot_of = paged_tokens(np.asarray(kv_indices), base, kv_len, page_size)
    return cache[page_of, slot_of]


def valid_len(n_pages: int, last_page_len: int, page_size: int) -> int:
    return min(max(n_pages - 1, 0) * page_size + max(last_page_len, 0), n_pages * page_size)


def split_ranges(n_tokens: int, tile: int, split: int) -> list:
    """``[(tile0, trip)]`` per split."""
    n_tiles = -(-n_tokens // tile)
    per = -(-n_tiles // split)
    return [(s * per, max(min(per, n_tiles - s * per), 0)) for s in range(split)]


def attend(q: np.ndarray, k: np.ndarray, v: np.ndarray, scale: float):
    """``q`` (heads, d), ``k``/``v`` (n_kv, heads, d), all float32 -> (out (heads, d), lse2 (heads,))."""
    logits = np.einsum("hd,khd->hk", q, k, dtype=np.float32) * np.float32(scale)
    m = logits.max(axis=-1, keepdims=True)
    e = np.exp(logits - m, dtype=np.float32)
    s = e.sum(axis=-1, keepdims=True, dtype=np.float32)
    w = e / s
    lse2 = (m[:, 0] + np.log(s[:, 0], dtype=np.float32)) / np.float32(math.log(2.0))
    out = np.einsum("hk,khd->hd", w, v, dtype=np.float32)
    return out, lse2


def decode(q, k_cache, v_cache, kv_indptr, kv_indices, kv_lens, page_size, sm_scale, out_dtype="float16"):
    """-> ``(out (batch, hq, d) float32 on out_dtype's grid, lse (batch, hq) float32)``."""
    qf, kc, vc = to_f32(q), to_f32(k_cache), to_f32(v_cache)
    indptr = np.asarray(kv_indptr.cpu() if hasattr(kv_indptr, "cpu") else kv_indptr, dtype=np.int64)
    indices = np.asarray(kv_indices.cpu() if hasattr(kv_indices, "cpu") else kv_indices, dtype=np.int64)
    batch, hq, d = qf.shape
    hkv = kc.shape[2]
    group = hq // hkv
    out = np.zeros((batch, hq, d), dtype=np.float32)
    lse = np.full((batch, hq), -np.inf, dtype=np.float32)
    for b, n in enumerate(kv_lens):
        n = int(n)
        if n <= 0:
            continue
        kk = np.repeat(gather(kc, indices, int(indptr[b]), n, page_size), group, axis=1)
        vv = np.repeat(gather(vc, indices, int(indptr[b]), n, page_size), group, axis=1)
        o, l = attend(qf[b], kk, vv, sm_scale)
        out[b] = round_to_dtype(o, out_dtype)
        lse[b] = l
    return out, lse


def mla_attend(qn: np.ndarray, qp: np.ndarray, kc: np.ndarray, kp: np.ndarray, scale: float):
    """``qn`` (heads, ckv), ``qp`` (heads, kpe), ``kc`` (n_kv, ckv), ``kp`` (n_kv, kpe), all float32
    -> (out (heads, ckv), lse2 (heads,))."""
    logits = (np.einsum("hd,kd->hk", qn, kc, dtype=np.float32)
              + np.einsum("hd,kd->hk", qp, kp, dtype=np.float32)) * np.float32(scale)
    m = logits.max(axis=-1, keepdims=True)
    e = np.exp(logits - m, dtype=np.float32)
    s = e.sum(axis=-1, keepdims=True, dtype=np.float32)
    lse2 = (m[:, 0] + np.log(s[:, 0], dtype=np.float32)) / np.float32(math.log(2.0))
    return np.einsum("hk,kd->hd", e / s, kc, dtype=np.float32), lse2


def mla_decode(q_nope, q_pe, ckv_cache, kpe_cache, kv_indptr, kv_indices, kv_lens, sm_scale, out_dtype="bfloat16"):
    """-> ``(out (batch, heads, ckv) float32 on out_dtype's grid, lse (batch, heads) float32)``."""
    qn, qp, cc, pc = to_f32(q_nope), to_f32(q_pe), to_f32(ckv_cache), to_f32(kpe_cache)
    indptr = np.asarray(kv_indptr.cpu() if hasattr(kv_indptr, "cpu") else kv_indptr, dtype=np.int64)
    indices = np.asarray(kv_indices.cpu() if hasattr(kv_indices, "cpu") else kv_indices, dtype=np.int64)
    batch, heads, ckv = qn.shape
    out = np.zeros((batch, heads, ckv), dtype=np.float32)
    lse = np.full((batch, heads), -np.inf, dtype=np.float32)
    for b, n in enumerate(kv_lens):
        n = int(n)
        if n <= 0:
            continue
        rows = indices[int(indptr[b]):int(indptr[b]) + n]
        o, l = mla_attend(qn[b], qp[b], cc[rows, 0], pc[rows, 0], sm_scale)
        out[b] = round_to_dtype(o, out_dtype)
        lse[b] = l
    return out, lse


def causal_keep(q_len: int, kv_len: int) -> np.ndarray:
    q_pos = np.arange(q_len)[:, None]
    kv_pos = np.arange(kv_len)[None, :]
    return kv_pos <= (kv_len - q_len) + q_pos


def _attend_masked(q, k, v, scale, keep):
    """``q`` (n_q, heads, d), ``k``/``v`` (n_kv, heads, d) float32, ``keep`` (n_q, n_kv) bool ->
    out (n_q, heads, d), lse2 (n_q, heads); a row with nothing kept gives 0 and -inf."""
    logits = np.einsum("qhd,khd->qhk", q, k, dtype=np.float32) * np.float32(scale)
    logits = np.where(keep[:, None, :], logits, -np.inf).astype(np.float32)
    m = logits.max(axis=-1, keepdims=True)
    dead = np.isneginf(m)
    e = np.exp(logits - np.where(dead, 0.0, m), dtype=np.float32)
    s = e.sum(axis=-1, keepdims=True, dtype=np.float32)
    w = np.where(dead, 0.0, e / np.where(dead, 1.0, s)).astype(np.float32)
    with np.errstate(divide="ignore"):
        lse2 = np.where(dead[..., 0], -np.inf, (m[..., 0] + np.log(s[..., 0], dtype=np.float32)) / np.float32(math.log(2.0)))
    return np.einsum("qhk,khd->qhd", w, v, dtype=np.float32), lse2.astype(np.float32)


def prefill(q, k, v, qo_indptr, kv_indptr, kv_indices, q_lens, kv_lens, sm_scale, out_dtype="bfloat16"):
    """Causal prefill of ragged queries.  ``kv_indices`` is the token table (then ``k``/``v`` are
    caches (num_pages, 1, kv_heads, d)) or None (packed keys (total_kv, kv_heads, d))."""
    qf, kf, vf = to_f32(q), to_f32(k), to_f32(v)
    as_i64 = lambda a: np.asarray(a.cpu() if hasattr(a, "cpu") else a, dtype=np.int64)  # noqa: E731
    qo, kvp = as_i64(qo_indptr), as_i64(kv_indptr)
    idx = None if kv_indices is None else as_i64(kv_indices)
    total_q, hq, d = qf.shape
    hkv = kf.shape[-2]
    group = hq // hkv
    out = np.zeros((total_q, hq, d), dtype=np.float32)
    lse = np.full((total_q, hq), -np.inf, dtype=np.float32)
    for r, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        ql, kl = int(ql), int(kl)
        if ql <= 0 or kl <= 0:
            continue
        qs = int(qo[r])
        if idx is None:
            kk, vv = kf[int(kvp[r]):int(kvp[r]) + kl], vf[int(kvp[r]):int(kvp[r]) + kl]
        else:
            rows = idx[int(kvp[r]):int(kvp[r]) + kl]
            kk, vv = kf[rows, 0], vf[rows, 0]
        o, l = _attend_masked(qf[qs:qs + ql], np.repeat(kk, group, axis=1), np.repeat(vv, group, axis=1), sm_scale,
                              causal_keep(ql, kl))
        out[qs:qs + ql] = round_to_dtype(o, out_dtype)
        lse[qs:qs + ql] = l
    return out, lse


def mla_prefill(q_nope, q_pe, ckv_cache, kpe_cache, qo_indptr, kv_indptr, kv_indices, q_lens, kv_lens, sm_scale,
                out_dtype="bfloat16"):
    """-> ``(out (total_q, heads, ckv) float32 on out_dtype's grid, lse (total_q, heads) float32)``."""
    qn, qp, cc, pc = to_f32(q_nope), to_f32(q_pe), to_f32(ckv_cache), to_f32(kpe_cache)
    as_i64 = lambda a: np.asarray(a.cpu() if hasattr(a, "cpu") else a, dtype=np.int64)  # noqa: E731
    qo, kvp, idx = as_i64(qo_indptr), as_i64(kv_indptr), as_i64(kv_indices)
    total_q, heads, ckv = qn.shape
    out = np.zeros((total_q, heads, ckv), dtype=np.float32)
    lse = np.full((total_q, heads), -np.inf, dtype=np.float32)
    for r, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        ql, kl = int(ql), int(kl)
        if ql <= 0 or kl <= 0:
            continue
        qs = int(qo[r])
        rows = idx[int(kvp[r]):int(kvp[r]) + kl]
        # scores of both terms as one product over joined features; values = the latent rows
        q_joined = np.concatenate([qn[qs:qs + ql], qp[qs:qs + ql]], axis=-1)
        k_joined = np.concatenate([cc[rows, 0], pc[rows, 0]], axis=-1)[:, None, :].repeat(heads, axis=1)
        v_latent = cc[rows, 0][:, None, :].repeat(heads, axis=1)
        o, l = _attend_masked(q_joined, k_joined, v_latent, sm_scale, causal_keep(ql, kl))
        out[qs:qs + ql] = round_to_dtype(o, out_dtype)
        lse[qs:qs + ql] = l
    return out, lse
