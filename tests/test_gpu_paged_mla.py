"""GPU parity of the paged MLA decode layer (token table, page size 1) against the numpy oracle:
the single kernel and the chunked split pair, ragged request lengths around the 32-token step
and the 256-entry table window, empty requests, a rising maximum (the softmax reference is
raised several times), more than one 16-head group, and the registry operator's workloads."""

import numpy as np
import pytest
import torch

from cleave_amd.codegen import HipCodeGen
from cleave_amd.dynamic import reference as dref
from cleave_amd.dynamic.paging import MLA_PAGED_PREFILL_CAUSAL, CombineTiling, DenseMLA, MLASpec, build_split_decode
from cleave_amd.dynamic.paging.apply import _mla_outputs, _mla_params, _mla_plan
from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code
from oracle import paged_oracle

pytestmark = pytest.mark.gpu


def mla_kernel(heads=16, ckv=512, kpe=64, split=None, chunk_pages=-1, dtype="bfloat16", stages=2, ksplit=1):
    spec = MLASpec(num_qo_heads=heads)
    dense = DenseMLA(heads, ckv, kpe, dtype, dtype, chunk_pages=chunk_pages, stages=stages, ksplit=ksplit)
    if split:
        src = HipCodeGen().gen(build_split_decode(spec, dense, split, CombineTiling(split=split)))
    else:
        params, ops = _mla_params(spec, dense)
        outs, out_ops = _mla_outputs(spec, dense)
        src = HipCodeGen().gen(_mla_plan(spec, dense, "main", params + outs, {**ops, **out_ops}))
    loaded = _load_main_kernel_from_code(src)
    return _compile(loaded, loaded.manifest["out_idx"])


def workload(lens, num_pages, heads=16, ckv=512, kpe=64, pad=0, scale=None, seed=0):
    n_idx = sum(lens) + pad
    return dref.mla_paged_decode_inputs((len(lens), heads, ckv, kpe, num_pages, n_idx), lens, scale=scale,
                                        device="cpu", seed=seed)


def check(kernel, args, lens, what):
    print(f"paged mla case {what} lens={lens}", flush=True)
    out, lse = kernel(*[a.cuda() if isinstance(a, torch.Tensor) else a for a in args])
    torch.cuda.synchronize()
    got_o, got_l = out.float().cpu().numpy(), lse.cpu().numpy()
    want_o, want_l = paged_oracle.mla_decode(*args[:6], lens, args[6], out_dtype="bfloat16")
    np.testing.assert_allclose(got_o, want_o, rtol=1e-2, atol=1e-2)
    live = np.isfinite(want_l)
    np.testing.assert_allclose(got_l[live], want_l[live], rtol=1e-3, atol=1e-3)
    assert np.all(np.isneginf(got_l[~live])), "an empty request must give lse = -inf"
    assert np.all(got_o[np.array(lens) == 0] == 0), "an empty request must give out = 0"


LENS = [1, 31, 32, 33, 0, 255, 256, 257, 700, 5, 0, 1100]


@pytest.mark.parametrize("split,chunk_pages", [(None, -1), (4, -1), (4, 32), (4, 45), (4, 300)])
def test_paged_mla_decode(split, chunk_pages):
    args = workload(LENS, num_pages=5000, pad=7)
    check(mla_kernel(split=split, chunk_pages=chunk_pages), args, LENS, f"split={split} chunk={chunk_pages}")


@pytest.mark.parametrize("split,chunk_pages", [(None, -1), (4, 45), (4, 300)])
def test_paged_mla_decode_three_images(split, chunk_pages):
    """The rows of two steps in flight behind the one in the matrix cores: requests of one, two and
    three steps (fewer steps than images), around the 256-entry table window, empty ones."""
    lens = LENS + [64, 65, 96, 97, 513]
    args = workload(lens, num_pages=6000, pad=7)
    check(mla_kernel(split=split, chunk_pages=chunk_pages, stages=3), args, lens, f"stages=3 split={split} chunk={chunk_pages}")


def test_paged_mla_decode_two_waves_share_a_request():
    """Two waves deal a request's steps out between them and the second folds into the first:
    requests of no, one, two and three steps (a wave without a step), odd and even step counts,
    around the 256-entry table window, and a second head group."""
    lens = LENS + [64, 65, 96, 97, 513]
    args = workload(lens, num_pages=6000, pad=7)
    check(mla_kernel(ksplit=2), args, lens, "ksplit=2")
    lens = [40, 300, 7]
    args = workload(lens, num_pages=900, heads=32, ckv=256, kpe=64)
    check(mla_kernel(heads=32, ckv=256, kpe=64, ksplit=2), args, lens, "h32 ckv256 ksplit=2")


def test_paged_mla_decode_rising_maximum():
    """Scores that keep growing along a request's tokens: the reference point is raised several
    times inside an item and the accumulators rescaled."""
    lens = [600, 90]
    args = workload(lens, num_pages=2000)
    qn, qp, ckv, kpe, indptr, idx, scale = args
    rows = idx[:sum(lens)].long()
    ramp = torch.cat([torch.linspace(0.1, 5.0, n) for n in lens]).reshape(-1, 1)
    direction = torch.sign(qn.float().mean(dim=(0, 1), keepdim=True)).reshape(1, -1)
    ckv = ckv.clone()
    ckv[rows, 0] = (ckv[rows, 0].float() * 0.2 + ramp * direction).to(ckv.dtype)
    args = [qn, qp, ckv, kpe, indptr, idx, scale]
    for split, stages, ksplit in ((None, 2, 1), (2, 2, 1), (None, 3, 1), (None, 2, 2)):
        check(mla_kernel(split=split, chunk_pages=128, stages=stages, ksplit=ksplit), args, lens,
              f"rising maximum split={split} stages={stages} ksplit={ksplit}")


def test_paged_mla_decode_lse_of_short_requests_is_not_rounded():
    """Requests of a handful of tokens show the element-type rounding of the weights in their lse
    unless the sum behind the lse is the one of the unrounded weights: single-item, chunked and
    key-sharing kernels alike (tolerance 2e-4 in log2 units; bf16 rounding would show up to 3e-3)."""
    lens = [2, 3, 1, 5, 2, 7, 3, 2]
    args = workload(lens, num_pages=200, heads=32, seed=11)
    want = paged_oracle.mla_decode(*args[:6], lens, args[6], out_dtype="bfloat16")[1]
    for kw in (dict(), dict(split=2), dict(split=4, chunk_pages=1), dict(ksplit=2), dict(stages=3)):
        print(f"paged mla short lse {kw}", flush=True)
        _, lse = mla_kernel(heads=32, **kw)(*[a.cuda() if isinstance(a, torch.Tensor) else a for a in args])
        np.testing.assert_allclose(lse.cpu().numpy(), want, rtol=0, atol=2e-4, err_msg=str(kw))


def test_paged_mla_decode_two_head_groups_and_other_widths():
    lens = [40, 300, 7]
    args = workload(lens, num_pages=900, heads=32, ckv=256, kpe=64)
    for split in (None, 3):
        check(mla_kernel(heads=32, ckv=256, kpe=64, split=split, chunk_pages=64), args, lens, f"h32 ckv256 split={split}")


def test_paged_mla_table_ids_outside_the_pool_are_clamped():
    """Padding entries of the table (and any id outside the pool) must never be dereferenced out
    of bounds: ids are clamped into the pool, and entries past a request's length are not read
    as tokens.  The padded tail holds huge ids here."""
    lens = [50, 10]
    args = workload(lens, num_pages=300, pad=20)
    args[5][sum(lens):] = 2 ** 30
    check(mla_kernel(), args, lens, "huge padding ids")


@pytest.mark.parametrize("axes", [(1, 989669, 8), (16, 989669, 457), (64, 989669, 9945)])
def test_registry_mla_operator_workloads(axes):
    """The registry operator at the reference's captured axes (the pool shrunk to what the
    table names plus slack: the pool size only changes which rows are gathered)."""
    from cleave_amd.dynamic import OPERATORS
    from cleave_amd.dynamic import workloads as wl

    op = OPERATORS["mla_paged_decode_h16_ckv512_kpe64_ps1"]
    batch, pool, n_idx, lens = wl.decode_lengths(op.name, axes, 1)
    pool = min(pool, 4 * n_idx + 64)
    args = dref.mla_paged_decode_inputs((batch, 16, 512, 64, pool, n_idx), lens, scale=op.scale, device="cpu")
    for split in (None, 8):
        check(mla_kernel(split=split), args, lens, f"registry axes {axes} split={split}")


def mla_prefill_kernel(heads=16, ckv=512, kpe=64, dtype="bfloat16", tok=4, stages=2, ksplit=1):
    spec = MLASpec(num_qo_heads=heads, kind=MLA_PAGED_PREFILL_CAUSAL, causal=True)
    spec.validate()
    dense = DenseMLA(heads, ckv, kpe, dtype, dtype, stages=stages, ksplit=ksplit)
    params, ops = _mla_params(spec, dense)
    outs, out_ops = _mla_outputs(spec, dense)
    loaded = _load_main_kernel_from_code(HipCodeGen().gen(_mla_plan(spec, dense, "main", params + outs, {**ops, **out_ops},
                                                                    tok=tok)))
    return _compile(loaded, loaded.manifest["out_idx"])


@pytest.mark.parametrize("tok,stages,ksplit", [(1, 2, 1), (2, 2, 1), (4, 2, 1), (1, 3, 1), (2, 3, 1), (2, 4, 1), (4, 4, 1), (1, 2, 2)],
                         ids=lambda t: f"{t}")
@pytest.mark.parametrize("q_lens,kv_lens", [([1, 4, 5, 33, 0, 40, 7], [1, 4, 40, 33, 9, 300, 3]), ([6, 0, 3], [0, 5, 3]),
                                            ([90], [700]), ([3, 9], [2, 5])])
def test_paged_mla_causal_prefill(q_lens, kv_lens, tok, stages, ksplit):
    """Ragged query rows, one, two or four query tokens per item (one wave each, sharing the
    item's two to four key images), or two waves on one token dealing its steps out between them: equal lengths, a cached prefix, windows shorter than the query run (fully
    masked rows beside live ones in one item), requests without queries or without keys, a long
    prefix (table windows reloaded), items cut by request boundaries."""
    tq, tk = sum(q_lens), sum(kv_lens)
    args = dref.mla_paged_prefill_inputs((16, 512, 64, 4 * tk + 64, tk + 3, tq), q_lens, kv_lens, device="cpu")
    print(f"paged mla prefill q_lens={q_lens} kv_lens={kv_lens} tok={tok} stages={stages} ksplit={ksplit}", flush=True)
    out, lse = mla_prefill_kernel(tok=tok, stages=stages, ksplit=ksplit)(*[a.cuda() if isinstance(a, torch.Tensor) else a for a in args])
    torch.cuda.synchronize()
    got_o, got_l = out.float().cpu().numpy(), lse.cpu().numpy()
    want_o, want_l = paged_oracle.mla_prefill(*args[:7], q_lens, kv_lens, args[7])
    np.testing.assert_allclose(got_o, want_o, rtol=1e-2, atol=1e-2)
    live = np.isfinite(want_l)
    np.testing.assert_allclose(got_l[live], want_l[live], rtol=1e-3, atol=1e-3)
    assert np.all(np.isneginf(got_l[~live])) and np.all(got_o[~live.any(axis=1)] == 0)
