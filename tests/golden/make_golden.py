"""Writes tests/golden/*.npz: small input/expected vectors computed in float64 from closed forms
that do not share code with the oracle or the package (plain numpy expressions, written out).

    python tests/golden/make_golden.py

Closed forms follow the reference's own tests: x @ w (tests/frontend/test_program.py:26-32),
x * rsqrt(mean(x^2) [+ eps]) [* gamma] @ w (:35-40), softmax(q k^T / sqrt(d)) v with the kv heads
repeat-interleaved over the group (:43-52), MLA scores q kv^T + q_pe k_pe^T (demo/mla_decode.py:9-13),
and the paged gather cache[page_of, slot_of] (python/cleave/dynamic/reference.py:143-152,192-193).
Inputs are stored in the dtype grid they will be fed in (float16 values as float32 arrays).
"""

import math
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def f16(x):
    return np.asarray(x, dtype=np.float64).astype(np.float16).astype(np.float64)


def bf16(x):
    x = np.asarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    r = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32).astype(np.float64)


def softmax64(s):
    e = np.exp(s - s.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


def main():
    rng = np.random.default_rng(20240521)
    # matmul
    x, w = f16(rng.uniform(-1, 1, (8, 32)) / math.sqrt(32)), f16(rng.uniform(-1, 1, (32, 16)) / math.sqrt(32))
    np.savez(os.path.join(HERE, "matmul.npz"), x=x, w=w, y=x @ w)
    # rmsnorm -> matmul with gamma and eps
    x, g, w = f16(rng.normal(size=(4, 64))), f16(1 + 0.1 * rng.normal(size=(1, 64))), f16(rng.normal(size=(64, 24)) / 8)
    y = (x / np.sqrt((x * x).mean(-1, keepdims=True) + 1e-6) * g) @ w
    np.savez(os.path.join(HERE, "rmsnorm_matmul.npz"), x=x, gamma=g, w=w, y=y, eps=1e-6)
    # GQA attention: 6 query heads over 2 kv heads, exact softmax
    q, k, v = f16(rng.normal(size=(6, 3, 16))), f16(rng.normal(size=(2, 40, 16))), f16(rng.normal(size=(2, 40, 16)))
    kk, vv = np.repeat(k, 3, axis=0), np.repeat(v, 3, axis=0)
    o = softmax64(q @ kk.transpose(0, 2, 1) / 4.0) @ vv
    np.savez(os.path.join(HERE, "gqa_attention.npz"), q=q, k=k, v=v, o=o)
    # MLA decode
    q, kv = bf16(0.5 * rng.normal(size=(2, 16, 32))), bf16(0.5 * rng.normal(size=(2, 20, 32)))
    qp, kp = bf16(0.5 * rng.normal(size=(2, 16, 8))), bf16(0.5 * rng.normal(size=(2, 20, 8)))
    s = (q @ kv.transpose(0, 2, 1) + qp @ kp.transpose(0, 2, 1)) * (40 ** -0.5)
    np.savez(os.path.join(HERE, "mla_decode.npz"), q=q, kv=kv, q_pe=qp, k_pe=kp, o=softmax64(s) @ kv, scale=40 ** -0.5)
    # paged GQA decode: page 4, 3 requests (one empty), 4 query heads over 2 kv heads
    page, lens, hq, hkv, d, pool = 4, [6, 0, 9], 4, 2, 8, 11
    pages = [-(-n // page) for n in lens]
    table = rng.permutation(pool)[:sum(pages)].astype(np.int32)
    indptr = np.concatenate([[0], np.cumsum(pages)]).astype(np.int32)
    last = np.array([n - (p - 1) * page if p else 0 for n, p in zip(lens, pages)], dtype=np.int32)
    q = f16(rng.normal(size=(3, hq, d)))
    kc, vc = f16(rng.normal(size=(pool, page, hkv, d))), f16(rng.normal(size=(pool, page, hkv, d)))
    out, lse = np.zeros((3, hq, d)), np.full((3, hq), -np.inf)
    gathered = {}
    for b, n in enumerate(lens):
        if n == 0:
            continue
        rows_k = np.stack([kc[table[indptr[b] + t // page], t % page] for t in range(n)])   # (n, hkv, d)
        rows_v = np.stack([vc[table[indptr[b] + t // page], t % page] for t in range(n)])
        gathered[f"k{b}"], gathered[f"v{b}"] = rows_k, rows_v
        for h in range(hq):
            s = rows_k[:, h // (hq // hkv)] @ q[b, h] * d ** -0.5
            out[b, h] = softmax64(s) @ rows_v[:, h // (hq // hkv)]
            lse[b, h] = (s.max() + np.log(np.exp(s - s.max()).sum())) / math.log(2.0)
    np.savez(os.path.join(HERE, "paged_decode.npz"), q=q, k_cache=kc, v_cache=vc, kv_indptr=indptr, kv_indices=table,
             kv_last_page_len=last, lens=np.array(lens), out=out, lse=lse, scale=d ** -0.5, page=page, **gathered)
    print("golden vectors written to", HERE)


if __name__ == "__main__":
    main()
