"""Pins of the numpy oracle: golden vectors (float64 closed forms), brute force on tiny inputs,
invariants.  A dropped term, a wrong sign or index, or a transposed operand fails one of them."""

import math
from pathlib import Path

import numpy as np
import pytest
import torch

import cleave_amd.lang as cl
from cleave_amd.frontend import Program
from oracle import paged_oracle, program_oracle as po
from cleave_amd import examples as C

GOLD = Path(__file__).parent / "golden"


def load(name):
    return {k: v for k, v in np.load(GOLD / name).items()}


def t(a, dtype=torch.float16):
    return torch.tensor(np.asarray(a, dtype=np.float32)).to(dtype)


def close(got, want, tol):
    np.testing.assert_allclose(np.asarray(got, dtype=np.float64), want, rtol=tol, atol=tol)


# ----------------------------------------------------------------------------- golden vectors
def test_golden_matmul():
    g = load("matmul.npz")
    prog = C.matmul.trace(cl.f16, M=8, K=32, N=16)
    close(po.evaluate(prog, [t(g["x"]), t(g["w"])], round_outputs=False)[0], g["y"], 1e-5)


def test_golden_rmsnorm_matmul_with_gamma_and_eps():
    g = load("rmsnorm_matmul.npz")
    prog = C.rmsnorm_matmul.trace(cl.f16, M=4, K=64, N=24)
    close(po.evaluate(prog, [t(g["x"]), t(g["gamma"]), t(g["w"])], round_outputs=False)[0], g["y"], 2e-5)
    # and the rounded output is exactly the nearest float16 of the float32 result
    y16 = po.evaluate(prog, [t(g["x"]), t(g["gamma"]), t(g["w"])])[0]
    assert np.array_equal(y16, y16.astype(np.float16).astype(np.float32))


def test_golden_gqa_attention_exact_and_shift_programs_agree():
    g = load("gqa_attention.npz")
    shapes = dict(HQ=6, HKV=2, SQ=3, SKV=40, D=16)
    ins = [t(g["q"]), t(g["k"]), t(g["v"])]
    exact = po.evaluate(C.gqa_decode_exact.trace(cl.f16, **shapes), ins, round_outputs=False)[0]
    close(exact, g["o"], 2e-5)
    shift = po.evaluate(C.gqa_decode_shift.trace(cl.f16, **shapes), ins, round_outputs=False)[0]
    close(shift, g["o"], 2e-5)          # softmax is shift invariant


def test_golden_mla_decode():
    g = load("mla_decode.npz")
    @cleave_amd_jit
    def mla(q: cl.Tensor["B", "H", "D"], kv: cl.Tensor["B", "SKV", "D"], q_pe: cl.Tensor["B", "H", "PE"],
            k_pe: cl.Tensor["B", "SKV", "PE"]):
        return cl.softmax((q @ kv.mT + q_pe @ k_pe.mT) * (40 ** -0.5), dim=-1) @ kv
    prog = mla.trace(cl.bf16, B=2, H=16, D=32, PE=8, SKV=20)
    ins = [t(g[k], torch.bfloat16) for k in ("q", "kv", "q_pe", "k_pe")]
    close(po.evaluate(prog, ins, round_outputs=False)[0], g["o"], 3e-5)


def cleave_amd_jit(fn):
    import cleave_amd

    return cleave_amd.jit(fn)


def test_golden_paged_decode_and_gather():
    g = load("paged_decode.npz")
    lens, page = g["lens"].tolist(), int(g["page"])
    out, lse = paged_oracle.decode(g["q"], g["k_cache"], g["v_cache"], g["kv_indptr"], g["kv_indices"], lens, page,
                                   float(g["scale"]), out_dtype="float32")
    close(out, g["out"], 2e-5)
    live = np.isfinite(g["lse"])
    close(lse[live], g["lse"][live], 2e-5)
    assert np.all(np.isneginf(lse[~live])) and np.all(out[1] == 0)      # the empty request
    for b, n in enumerate(lens):
        if n:
            got = paged_oracle.gather(g["k_cache"], g["kv_indices"], int(g["kv_indptr"][b]), n, page)
            assert np.array_equal(got, g[f"k{b}"])                       # the gather is bit exact


# ----------------------------------------------------------------------------- brute force / invariants
def test_every_record_kind_against_scalar_loops():
    p = Program("p", cl.f32)
    a, b = p.input("a", [3, 4]), p.input("b", [3, 1])
    p.output(a - b), p.output(b - a), p.output(2.0 - a), p.output(a / b), p.output(3.0 / a)
    p.output(a.max(-1, keepdim=True)), p.output(a.sum(0, keepdim=True)), p.output((a * a).sqrt())
    p.output(a.silu()), p.output(a.exp()), p.output(a * 0.5 + 1.0)
    rng = np.random.default_rng(0)
    A, B = rng.uniform(0.5, 2, (3, 4)).astype(np.float32), rng.uniform(0.5, 2, (3, 1)).astype(np.float32)
    got = po.evaluate(p, [A, B])
    want = [A - B, B - A, 2 - A, A / B, 3 / A, A.max(-1, keepdims=True), A.sum(0, keepdims=True), np.abs(A),
            A / (1 + np.exp(-A)), np.exp(A), A * 0.5 + 1]
    for x, y in zip(got, want):
        close(x, y.astype(np.float64), 1e-6)


def test_demo_programs_against_float64_restatements_and_identities():
    """The oracle on the later operators (SwiGLU, LoRA, matmul + row sum, QK-norm attention, attention
    with unlike key / value widths): against float64 formulas written from the reference's graph
    docstrings (``tests/_graphs.py:150-160, 403-436, 438-480, 542-640``), and against what the
    mathematics fixes -- the row sum of a product is the product with the row sums of B; SwiGLU is
    linear in the bare weight; LoRA with a zero factor is the base product; RMS-normalised rows
    do not change when a row is scaled."""
    rng = np.random.default_rng(7)
    f = lambda *s: rng.normal(size=s).astype(np.float32)          # noqa: E731
    d = lambda x: x.astype(np.float64)                            # noqa: E731
    x, wu, wg = f(5, 12), f(12, 7), f(12, 7)
    prog = C.swiglu.trace(cl.f32, M=5, K=12, N=7)
    got = po.evaluate(prog, [x, wu, wg])[0]
    gate = d(x) @ d(wg)
    close(got, (d(x) @ d(wu)) * gate / (1 + np.exp(-gate)), 1e-5)
    close(po.evaluate(prog, [x, 3 * wu, wg])[0], 3 * d(got), 1e-5)                       # linear in w_up
    a, b = f(12, 4), f(4, 7)
    prog = C.lora.trace(cl.f32, M=5, K=12, N=7, R=4)
    close(po.evaluate(prog, [x, wu, a, b])[0], d(x) @ d(wu) + (d(x) @ d(a)) @ d(b), 1e-5)
    close(po.evaluate(prog, [x, wu, a, 0 * b])[0], d(x) @ d(wu), 1e-5)                   # zero factor: the base product
    prog = C.matmul_rowsum.trace(cl.f32, M=5, K=12, N=7)
    got = po.evaluate(prog, [x, wu])[0]
    assert got.shape == (5, 1)
    close(got[:, 0], d(x) @ d(wu).sum(1), 1e-5)                                          # (x w) 1 = x (w 1)
    q, k, v = f(4, 6, 8), f(2, 9, 8), f(2, 9, 8)
    prog = C.qknorm.trace(cl.f32, HQ=4, HKV=2, SQ=6, SKV=9, D=8)
    got = po.evaluate(prog, [q, k, v])[0]
    nrm = lambda t: d(t) / np.sqrt((d(t) ** 2).mean(-1, keepdims=True) + 1e-6)           # noqa: E731
    for h in range(4):
        s_ = (nrm(q[h]) @ nrm(k[h // 2]).T) / np.sqrt(8)
        w_ = np.exp(s_ - s_.max(-1, keepdims=True))
        close(got[h], (w_ / w_.sum(-1, keepdims=True)) @ d(v[h // 2]), 1e-5)
    q2, k2 = q.copy(), k.copy()
    q2[1, 3] *= 5.0
    k2[0, 2] *= 0.25
    close(po.evaluate(prog, [q2, k2, v])[0], d(got), 1e-4)                               # scale-free rows
    kk, vv = f(3, 9, 12), f(3, 9, 4)
    prog = C.mla_prefill.trace(cl.f32, H=3, SQ=6, SKV=9, DK=12, DV=4)
    got = po.evaluate(prog, [f(3, 6, 12) * 0 + 1, kk, vv])[0]                            # equal queries: rows of a head agree
    close(got[:, 0], d(got[:, 5]), 1e-6)
    assert got.shape == (3, 6, 4)


def test_grouped_matmul_is_repeat_interleave_not_tile():
    rng = np.random.default_rng(1)
    a, b = rng.normal(size=(6, 2, 4)).astype(np.float32), rng.normal(size=(2, 4, 5)).astype(np.float32)
    got = po.grouped_matmul(a, b)
    for h in range(6):
        close(got[h], a[h].astype(np.float64) @ b[h // 3], 1e-5)       # head h pairs with kv head h // group
    got_t = po.grouped_matmul(a, np.swapaxes(b, -1, -2).copy(), trans_b=True)
    close(got_t, got, 1e-6)


def test_bfloat16_rounding_matches_torch_bit_for_bit():
    x = np.random.default_rng(2).normal(size=4096).astype(np.float32) * 37
    x[:4] = [0.0, -0.0, 1.00390625, 3.3895314e38]                      # a tie and a near-overflow
    want = torch.tensor(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(po.round_to_dtype(x, "bfloat16"), want)
    assert np.array_equal(po.round_to_dtype(x, "float16"), torch.tensor(x).to(torch.float16).float().numpy())


def test_page_permutation_leaves_paged_decode_unchanged():
    lens = [5, 12, 7]
    args = C.paged_workload(lens, page_size=4, num_pages=16, hq=4, hkv=2, d=8)
    base = paged_oracle.decode(*args[:5], lens, 4, args[-1])
    perm = torch.randperm(16, generator=torch.Generator().manual_seed(3))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(16)
    moved = paged_oracle.decode(args[0], args[1][perm], args[2][perm], args[3], inv[args[4].long()], lens, 4, args[-1])
    assert np.array_equal(base[0], moved[0]) and np.array_equal(base[1], moved[1])


@pytest.mark.parametrize("n_pages,last,page,want", [(0, 0, 64, 0), (1, 17, 64, 17), (3, 64, 64, 192), (3, 1, 64, 129),
                                                      (2, 999, 64, 128), (2, -5, 64, 64), (0, 9, 64, 0)])
def test_valid_len_formula(n_pages, last, page, want):
    assert paged_oracle.valid_len(n_pages, last, page) == want


@pytest.mark.parametrize("n_tokens,tile,split", [(0, 64, 8), (1, 64, 8), (64 * 7 + 3, 64, 8), (16384, 32, 16), (100, 32, 32)])
def test_every_kv_tile_is_owned_by_exactly_one_split(n_tokens, tile, split):
    owned = []
    for t0, trip in paged_oracle.split_ranges(n_tokens, tile, split):
        owned += list(range(t0, t0 + trip))
    assert owned == list(range(-(-n_tokens // tile)))


def test_attend_lse_is_log2_of_the_partition_function():
    rng = np.random.default_rng(4)
    q, k, v = rng.normal(size=(2, 8)).astype(np.float32), rng.normal(size=(9, 2, 8)).astype(np.float32), \
        rng.normal(size=(9, 2, 8)).astype(np.float32)
    out, lse = paged_oracle.attend(q, k, v, 0.3)
    for h in range(2):
        s = (k[:, h].astype(np.float64) @ q[h]) * 0.3
        assert abs(lse[h] - math.log2(np.exp(s).sum())) < 1e-5
        close(out[h], (np.exp(s) / np.exp(s).sum()) @ v[:, h], 1e-5)


def test_program_reference_and_oracle_agree_on_the_graded_programs():
    """The frontend's own eager ``reference`` (torch) and the oracle (numpy) are independent
    restatements; they must agree on every graded program."""
    for name, (fn, dt, mk) in C.CASES.items():
        prog = fn.trace(dt, **C.SMALL[name])
        ins = mk(C.SMALL[name])
        want = prog.reference(*ins)[0].float().numpy()
        np.testing.assert_allclose(po.evaluate(prog, ins)[0], want, rtol=4e-3, atol=4e-3)


# ----------------------------------------------------------------------------- paged MLA decode
def _mla_case(lens, num_pages=300, heads=16, ckv=64, kpe=16, seed=5):
    rng = np.random.default_rng(seed)
    total = sum(lens)
    qn = rng.standard_normal((len(lens), heads, ckv)).astype(np.float32)
    qp = rng.standard_normal((len(lens), heads, kpe)).astype(np.float32)
    cc = rng.standard_normal((num_pages, 1, ckv)).astype(np.float32)
    pc = rng.standard_normal((num_pages, 1, kpe)).astype(np.float32)
    idx = rng.permutation(num_pages)[:total].astype(np.int32)
    ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    return qn, qp, cc, pc, ptr, idx


def test_mla_attend_is_attend_over_joined_features():
    """(q_nope c^T + q_pe r^T) is one product over the concatenated features, and the values are
    the latent part of the keys: MLA must equal the GQA oracle on the joined operands (a dropped
    term, a swapped operand or values taken from the rope part all break this)."""
    qn, qp, cc, pc, _, idx = _mla_case([23])
    rows = idx[:23]
    out, lse = paged_oracle.mla_attend(qn[0], qp[0], cc[rows, 0], pc[rows, 0], 0.17)
    q_joined = np.concatenate([qn[0], qp[0]], axis=-1)
    k_joined = np.concatenate([cc[rows, 0], pc[rows, 0]], axis=-1)[:, None, :].repeat(16, axis=1)
    v_latent = cc[rows, 0][:, None, :].repeat(16, axis=1)
    want_o, want_l = paged_oracle.attend(q_joined, k_joined, v_latent, 0.17)
    np.testing.assert_allclose(out, want_o, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(lse, want_l, rtol=1e-5, atol=1e-6)


def test_mla_decode_against_float64_brute_force_and_empty_requests():
    lens = [7, 0, 40, 1]
    qn, qp, cc, pc, ptr, idx = _mla_case(lens)
    out, lse = paged_oracle.mla_decode(qn, qp, cc, pc, ptr, idx, lens, 0.3, out_dtype="float32")
    for b, n in enumerate(lens):
        if n == 0:
            assert np.all(out[b] == 0) and np.all(np.isneginf(lse[b]))
            continue
        rows = idx[ptr[b]:ptr[b] + n]
        for h in range(16):
            logits = np.array([(np.dot(qn[b, h].astype(np.float64), cc[r, 0]) + np.dot(qp[b, h].astype(np.float64), pc[r, 0]))
                               * 0.3 for r in rows])
            w = np.exp(logits - logits.max())
            w /= w.sum()
            want = sum(wi * cc[r, 0].astype(np.float64) for wi, r in zip(w, rows))
            np.testing.assert_allclose(out[b, h], want, rtol=2e-5, atol=2e-6)
            assert lse[b, h] == pytest.approx(np.log2(np.exp(logits - logits.max()).sum()) + logits.max() / np.log(2), rel=1e-5)


def test_mla_decode_depends_on_the_table_only_through_the_rows_it_names():
    """Moving the named rows elsewhere in the pool and renaming them in the table changes nothing."""
    lens = [9, 30]
    qn, qp, cc, pc, ptr, idx = _mla_case(lens)
    out, lse = paged_oracle.mla_decode(qn, qp, cc, pc, ptr, idx, lens, 0.2)
    perm = np.random.default_rng(1).permutation(cc.shape[0])
    cc2, pc2 = np.empty_like(cc), np.empty_like(pc)
    cc2[perm], pc2[perm] = cc, pc
    out2, lse2 = paged_oracle.mla_decode(qn, qp, cc2, pc2, ptr, perm[idx].astype(np.int32), lens, 0.2)
    assert np.array_equal(out, out2) and np.array_equal(lse, lse2)


# ----------------------------------------------------------------------------- causal prefill
def _prefill_case(q_lens, kv_lens, hq=8, hkv=2, d=16, seed=9):
    rng = np.random.default_rng(seed)
    tq, tk = sum(q_lens), sum(kv_lens)
    q = rng.standard_normal((tq, hq, d)).astype(np.float32)
    k = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    v = rng.standard_normal((tk, hkv, d)).astype(np.float32)
    qo = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    kvp = np.concatenate([[0], np.cumsum(kv_lens)]).astype(np.int32)
    return q, k, v, qo, kvp


def test_causal_mask_is_a_prefix_length_per_query_row():
    """Row i of a request sees exactly the first kv_len - q_len + i + 1 keys: each row must equal
    plain attention over that prefix (an off-by-one or a start-aligned mask breaks this), rows
    whose prefix is empty are 0 / -inf, and a request with one query row is a decode."""
    q_lens, kv_lens = [5, 3, 1, 4], [9, 3, 6, 2]          # cached prefix, equal, decode-like, window shorter than the run
    q, k, v, qo, kvp = _prefill_case(q_lens, kv_lens)
    out, lse = paged_oracle.prefill(q, k, v, qo, kvp, None, q_lens, kv_lens, 0.25, out_dtype="float32")
    assert np.array_equal(paged_oracle.causal_keep(3, 5), np.array([[1, 1, 1, 0, 0], [1, 1, 1, 1, 0], [1, 1, 1, 1, 1]], bool))
    for r, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        for i in range(ql):
            n = kl - ql + i + 1
            row = qo[r] + i
            if n <= 0:
                assert np.all(out[row] == 0) and np.all(np.isneginf(lse[row]))
                continue
            kk = np.repeat(k[kvp[r]:kvp[r] + n], 4, axis=1)
            vv = np.repeat(v[kvp[r]:kvp[r] + n], 4, axis=1)
            want_o, want_l = paged_oracle.attend(q[row], kk, vv, 0.25)
            np.testing.assert_allclose(out[row], want_o, rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(lse[row], want_l, rtol=1e-5, atol=1e-6)


def test_token_table_and_packed_prefill_agree_and_mla_prefill_is_prefill_over_joined_features():
    q_lens, kv_lens = [4, 2], [7, 5]
    q, k, v, qo, kvp = _prefill_case(q_lens, kv_lens)
    out, lse = paged_oracle.prefill(q, k, v, qo, kvp, None, q_lens, kv_lens, 0.3)
    # the same rows scattered over a pool and named by a table
    perm = np.random.default_rng(2).permutation(40)[:k.shape[0]]
    kc, vc = np.zeros((40, 1, 2, 16), np.float32), np.zeros((40, 1, 2, 16), np.float32)
    kc[perm, 0], vc[perm, 0] = k, v
    out2, lse2 = paged_oracle.prefill(q, kc, vc, qo, kvp, perm.astype(np.int32), q_lens, kv_lens, 0.3)
    assert np.array_equal(out, out2) and np.array_equal(lse, lse2)
    # MLA: one "kv head" whose keys are [latent | rope] and whose values are the latent part
    rng = np.random.default_rng(4)
    qn, qp = rng.standard_normal((6, 4, 16)).astype(np.float32), rng.standard_normal((6, 4, 8)).astype(np.float32)
    cc, pc = rng.standard_normal((40, 1, 16)).astype(np.float32), rng.standard_normal((40, 1, 8)).astype(np.float32)
    idx = perm[:12].astype(np.int32)
    mo, ml = paged_oracle.mla_prefill(qn, qp, cc, pc, qo, kvp, idx, q_lens, kv_lens, 0.3, out_dtype="float32")
    for r, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        rows = idx[kvp[r]:kvp[r] + kl]
        for i in range(ql):
            n = kl - ql + i + 1
            o, l = paged_oracle.mla_attend(qn[qo[r] + i], qp[qo[r] + i], cc[rows[:n], 0], pc[rows[:n], 0], 0.3)
            np.testing.assert_allclose(mo[qo[r] + i], o, rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(ml[qo[r] + i], l, rtol=1e-5, atol=1e-6)
