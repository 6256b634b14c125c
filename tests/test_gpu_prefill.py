"""GPU parity of the causal prefill layers (ragged queries; keys through a token table or packed
per request) against the numpy oracle: request lengths around the 32-key step and the query
tile, a cached prefix (kv_len > q_len), key windows shorter than the query run (fully masked
rows: 0 / -inf), empty requests, both head groupings of the shipped operators."""

import numpy as np
import pytest
import torch

from cleave_amd.codegen import HipCodeGen
from cleave_amd.dynamic import reference as dref
from cleave_amd.dynamic.paging import PAGED_PREFILL_CAUSAL, RAGGED_PREFILL_CAUSAL, DenseAttention, PagingSpec
from cleave_amd.dynamic.paging.apply import _prefill_plan
from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code
from oracle import paged_oracle

pytestmark = pytest.mark.gpu


def prefill_kernel(ragged, hq=32, hkv=8, d=128, dtype="bfloat16", shared=False):
    kw = dict(cache_inputs=("K", "V")) if ragged else {}
    spec = PagingSpec(hq, hkv, kind=RAGGED_PREFILL_CAUSAL if ragged else PAGED_PREFILL_CAUSAL, causal=True, **kw)
    spec.validate()
    dense = DenseAttention(16, 32, d, hkv * 64, dtype, dtype, waves=hkv)
    loaded = _load_main_kernel_from_code(HipCodeGen().gen(_prefill_plan(spec, dense, shared=shared)))
    return _compile(loaded, loaded.manifest["out_idx"])


def check(ragged, q_lens, kv_lens, hq=32, hkv=8, d=128, pad=0, what="", shared=False):
    total_q, total_kv = sum(q_lens), sum(kv_lens)
    if ragged:
        args = dref.gqa_ragged_prefill_inputs((hq, hkv, d, total_q, total_kv), q_lens, kv_lens, device="cpu")
        table = None
    else:
        args = dref.gqa_paged_prefill_inputs((hq, hkv, d, 4 * total_kv + 50, total_kv + pad, total_q), q_lens, kv_lens,
                                             device="cpu")
        table = args[5]
    print(f"prefill case ragged={ragged} shared={shared} h{hq}/kv{hkv} q_lens={q_lens} kv_lens={kv_lens} {what}", flush=True)
    out, lse = prefill_kernel(ragged, hq, hkv, d, shared=shared)(*[a.cuda() if isinstance(a, torch.Tensor) else a for a in args])
    torch.cuda.synchronize()
    got_o, got_l = out.float().cpu().numpy(), lse.cpu().numpy()
    want_o, want_l = paged_oracle.prefill(args[0], args[1], args[2], args[3], args[4], table, q_lens, kv_lens, args[-1])
    np.testing.assert_allclose(got_o, want_o, rtol=1e-2, atol=1e-2)
    live = np.isfinite(want_l)
    np.testing.assert_allclose(got_l[live], want_l[live], rtol=1e-3, atol=1e-3)
    assert np.all(np.isneginf(got_l[~live])), "a row that sees no key must give lse = -inf"
    assert np.all(got_o[~live.any(axis=1)] == 0) if (~live.any(axis=1)).any() else True


Q_LENS = [1, 4, 5, 33, 0, 64, 7, 130]
KV_LENS = [1, 4, 40, 33, 9, 200, 3, 130]       # equal, cached prefix, no queries, window shorter than the run


SHARED = pytest.mark.parametrize("shared", [False, True], ids=["rows16", "lds128"])


@SHARED
@pytest.mark.parametrize("ragged", [False, True])
def test_causal_prefill(ragged, shared):
    check(ragged, Q_LENS, KV_LENS, pad=5, shared=shared)


@SHARED
@pytest.mark.parametrize("ragged", [False, True])
def test_causal_prefill_four_kv_heads(ragged, shared):
    """Eight query heads per kv head: two tokens per 16-row tile (16 per 128-row workgroup)."""
    check(ragged, [3, 70, 1, 0, 18], [3, 70, 50, 4, 6], hq=32, hkv=4, shared=shared)


@SHARED
def test_causal_prefill_requests_without_keys_or_queries(shared):
    check(False, [5, 0, 9], [0, 7, 9], what="kv_len 0 / q_len 0", shared=shared)
    check(True, [5, 0, 9], [0, 7, 9], what="kv_len 0 / q_len 0", shared=shared)


@SHARED
def test_causal_prefill_long_request(shared):
    """Requests long enough for many key steps per tile, hundreds of tiles and several 256-entry
    table windows."""
    check(True, [700], [700], shared=shared)
    check(False, [300, 2], [1000, 900], what="long cached prefix", shared=shared)
    check(False, [40, 33], [600, 290], what="table windows", shared=shared)


@pytest.mark.parametrize("seed", range(8))
def test_causal_prefill_random_shapes(seed):
    """Seeded random request lists (lengths 0..300, cached prefixes 0..500 or key windows shorter
    than the query run, 1..6 requests, either head grouping, either key form) through the
    LDS-shared kernel; every odd seed also through the 16-row kernel."""
    rng = np.random.default_rng(1000 + seed)
    n = int(rng.integers(1, 7))
    q_lens = [int(x) for x in rng.integers(0, 301, n)]
    kv_lens = [max(0, q + int(rng.integers(-40, 500))) if rng.random() < 0.8 else int(rng.integers(0, 60)) for q in q_lens]
    if sum(q_lens) == 0:
        q_lens[0] = 5
    if sum(kv_lens) == 0:
        kv_lens[0] = 7
    hkv = 8 if seed % 2 else 4
    ragged = bool((seed // 2) % 2)
    check(ragged, q_lens, kv_lens, hkv=hkv, pad=int(rng.integers(0, 9)), what=f"random seed {seed}", shared=True)
    if seed % 2:
        check(ragged, q_lens, kv_lens, hkv=hkv, what=f"random seed {seed}", shared=False)


@SHARED
@pytest.mark.parametrize("ragged", [False, True])
def test_causal_prefill_rising_maximum(ragged, shared):
    """Scores that grow along a request's keys: every row's softmax reference point is raised several
    times on the way (the cold path: sums and accumulators rescaled by a factor strictly between 0
    and 1), in both prefill kernels and both key layouts, a cached prefix included."""
    hq, hkv, d = 32, 8, 128
    q_lens, kv_lens = [40, 3, 150], [600, 500, 150]
    total_q, total_kv = sum(q_lens), sum(kv_lens)
    if ragged:
        args = dref.gqa_ragged_prefill_inputs((hq, hkv, d, total_q, total_kv), q_lens, kv_lens, device="cpu")
        table, rows = None, torch.arange(total_kv)
    else:
        args = dref.gqa_paged_prefill_inputs((hq, hkv, d, 4 * total_kv + 50, total_kv, total_q), q_lens, kv_lens, device="cpu")
        table = args[5]
        rows = table[:total_kv].long()
    q, k = args[0], args[1]
    q[..., 0] = 4.0
    ramp = torch.cat([torch.linspace(0.0, 35.0 * d ** 0.5 / (4 * 1.4427), n) for n in kv_lens])
    kk = k.reshape(-1, hkv, d)
    kk[rows, :, 0] = ramp.reshape(-1, 1).to(k.dtype)
    print(f"prefill rising maximum ragged={ragged} shared={shared}", flush=True)
    out, lse = prefill_kernel(ragged, hq, hkv, d, shared=shared)(*[a.cuda() if isinstance(a, torch.Tensor) else a for a in args])
    torch.cuda.synchronize()
    want_o, want_l = paged_oracle.prefill(args[0], args[1], args[2], args[3], args[4], table, q_lens, kv_lens, args[-1])
    np.testing.assert_allclose(out.float().cpu().numpy(), want_o, rtol=1e-2, atol=1e-2)
    np.testing.assert_allclose(lse.cpu().numpy(), want_l, rtol=1e-3, atol=2e-3)


@SHARED
@pytest.mark.parametrize("d", [64, 256])
def test_causal_prefill_other_head_widths(d, shared):
    """64-wide heads (half a 128-feature block of accumulators: the lanes past the width store nothing)
    and 256-wide ones (two blocks), both key forms, both kernels."""
    check(True, [5, 70, 1, 33], [5, 70, 50, 40], d=d, what=f"d={d}", shared=shared)
    check(False, [40, 3], [200, 35], d=d, pad=3, what=f"d={d}", shared=shared)
