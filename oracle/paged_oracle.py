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
                         request.
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
