"""GPU parity of the paged GQA decode layer: attention output against the numpy oracle, and the
block-table gather bit-exact through properties of the kernel's own output."""

import numpy as np
import pytest
import torch

from cleave_amd.codegen import HipCodeGen
from cleave_amd.dynamic.paging import (PAGED_DECODE_SLAB, CombineTiling, DenseAttention, PagingSpec,
                                       build_split_decode)
from cleave_amd.dynamic.paging.apply import _paged_outputs, _paged_params, _plan
from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code
from oracle import paged_oracle
from cleave_amd import examples as C

pytestmark = pytest.mark.gpu


def paged_kernel(page_size=64, hq=32, hkv=8, d=128, waves=4, split=None, dtype="float16", chunk_pages=0, prefetch=1,
                 skew=0, lockstep=False):
    kind = PAGED_DECODE_SLAB if page_size > 1 else "paged_decode"
    spec = PagingSpec(num_qo_heads=hq, num_kv_heads=hkv, kind=kind, page_size=page_size)
    dense = DenseAttention(16, 32, d, waves * 64, dtype, dtype, waves=waves, chunk_pages=chunk_pages, prefetch=prefetch,
                           skew=skew, lockstep=lockstep)
    if split:
        src = HipCodeGen().gen(build_split_decode(spec, dense, split, CombineTiling(split=split, cols=min(128, d))))
    else:
        params, ops = _paged_params(spec, dense)
        outs, out_ops = _paged_outputs(spec, dense)
        src = HipCodeGen().gen(_plan(spec, dense, "main", params + outs, {**ops, **out_ops}))
    loaded = _load_main_kernel_from_code(src)
    return _compile(loaded, loaded.manifest["out_idx"])


def run(kernel, args):
    out, lse = kernel(*[a.cuda() if isinstance(a, torch.Tensor) else a for a in args])
    torch.cuda.synchronize()
    return out.float().cpu().numpy(), lse.cpu().numpy()


def check(args, lens, page_size, **kw):
    kernel = paged_kernel(page_size=page_size, **kw)
    print(f"paged case lens={lens} page={page_size} {kw}", flush=True)
    got_o, got_l = run(kernel, args)
    want_o, want_l = paged_oracle.decode(*args[:5], lens, page_size, args[-1], out_dtype="float16")
    np.testing.assert_allclose(got_o, want_o, rtol=1e-2, atol=1e-2)
    live = np.isfinite(want_l)
    np.testing.assert_allclose(got_l[live], want_l[live], rtol=1e-3, atol=1e-3)
    assert np.all(np.isneginf(got_l[~live])), "an empty request must give lse = -inf"
    assert np.all(got_o[np.array(lens) == 0] == 0), "an empty request must give out = 0"


@pytest.mark.parametrize("split", [None, 4, 8])
@pytest.mark.parametrize("waves", [1, 4])
def test_paged_decode_ps64(split, waves):
    lens = [1, 63, 64, 65, 200, 777, 0, 1500]          # page tails, an empty request
    args = C.paged_workload(lens, page_size=64, num_pages=256)
    check(args, lens, 64, split=split, waves=waves)


@pytest.mark.parametrize("chunk_pages", [1, 4, 7, -1])
@pytest.mark.parametrize("prefetch,lockstep", [(1, False), (2, False), (1, True)])
def test_paged_decode_chunked_items(chunk_pages, prefetch, lockstep):
    """Work cut into items of chunk_pages pages: requests that end on, before and after a chunk
    boundary, an empty request between two others, a request inside one chunk; with the waves of an
    item free-running and meeting at a barrier before every step."""
    lens = [1, 63, 64, 65, 200, 777, 0, 1500, 4 * 64, 0, 3 * 64 + 1, 7 * 64 * 3]
    args = C.paged_workload(lens, page_size=64, num_pages=300)
    check(args, lens, 64, split=8, waves=8, chunk_pages=chunk_pages, prefetch=prefetch, lockstep=lockstep)


def test_paged_decode_chunked_other_head_counts():
    lens = [130, 9, 700]
    args = C.paged_workload(lens, page_size=16, num_pages=200, hq=16, hkv=4)
    check(args, lens, 16, split=4, waves=4, hq=16, hkv=4, chunk_pages=3)
    check(args, lens, 16, split=4, waves=4, hq=16, hkv=4, chunk_pages=2, lockstep=True)


def test_paged_decode_bf16_lse_of_short_requests_is_not_rounded():
    """At bf16 a request of a few tokens shows the rounding of its weights (2^-9 each) in the lse
    unless the row sum adds them up unrounded: single kernel, fixed split and chunked items, page
    sizes 1 and 64 (tolerance 2e-4; the rounded sum was off by up to 2e-3)."""
    lens = [2, 3, 1, 5, 2, 7, 3, 2, 4, 6]
    for page_size in (1, 64):
        args = C.paged_workload(lens, page_size=page_size, num_pages=40, hq=32, hkv=4, dtype=torch.bfloat16, seed=3)
        call = args if page_size > 1 else args[:5] + args[6:]
        want = paged_oracle.decode(*args[:5], lens, page_size, args[-1], out_dtype="bfloat16")[1]
        for kw in (dict(), dict(split=4), dict(split=4, chunk_pages=1, waves=4)):
            if kw.get("chunk_pages") and page_size == 1:
                continue
            print(f"paged bf16 short lse page={page_size} {kw}", flush=True)
            _, lse = run(paged_kernel(page_size=page_size, hq=32, hkv=4, dtype="bfloat16", **kw), call)
            np.testing.assert_allclose(lse, want, rtol=0, atol=2e-4, err_msg=f"page={page_size} {kw}")


@pytest.mark.parametrize("page_size", [1, 16])
def test_paged_decode_other_page_sizes(page_size):
    lens = [5, 33, 130, 64]
    args = C.paged_workload(lens, page_size=page_size, num_pages=400)
    if page_size == 1:
        args = args[:5] + args[6:]                     # one token per page reads no last_page_len
    kernel = paged_kernel(page_size=page_size, split=2)
    got_o, got_l = run(kernel, args)
    want_o, want_l = paged_oracle.decode(*args[:5], lens, page_size, args[-1])
    np.testing.assert_allclose(got_o, want_o, rtol=1e-2, atol=1e-2)
    np.testing.assert_allclose(got_l, want_l, rtol=1e-3, atol=1e-3)


def test_gather_is_bit_exact_one_hot():
    """With one-hot queries scaled so the softmax saturates on a single token, and V rows that
    encode their own (page, slot, head), the output *is* a gathered V row: any wrong page id,
    slot or head offset changes bits."""
    page, hkv, hq, d = 64, 8, 32, 128
    lens = [64 * 3 + 17, 64 * 5]
    args = C.paged_workload(lens, page_size=page, num_pages=97, seed=11)
    q, k_cache, v_cache, indptr, indices, last, scale = args
    num_pages = k_cache.shape[0]
    # K: token t of request b has a large component in feature (t % d); Q picks feature f.
    k_cache.zero_()
    ids = torch.arange(num_pages * page * hkv).reshape(num_pages, page, hkv)
    v_cache.copy_(((ids % 2039).to(torch.float16) / 8.0)[..., None].expand(-1, -1, -1, d))
    targets = []
    for b, n in enumerate(lens):
        t = (7 * b + 40) % n
        pg = int(indices[int(indptr[b]) + t // page])
        k_cache[pg, t % page, :, 3] = 60.0
        targets.append((pg, t % page))
    q.zero_()
    q[:, :, 3] = 60.0
    kernel = paged_kernel(page_size=page, split=4)
    got_o, _ = run(kernel, [q, k_cache, v_cache, indptr, indices, last, 1.0])
    for b, (pg, slot) in enumerate(targets):
        for h in range(hq):
            want = v_cache[pg, slot, h // (hq // hkv)].float().numpy()
            assert np.array_equal(got_o[b, h], want), (b, h)


def test_page_permutation_leaves_output_bit_identical():
    lens = [300, 129, 64]
    args = C.paged_workload(lens, page_size=64, num_pages=64, seed=9)
    q, k_cache, v_cache, indptr, indices, last, scale = args
    kernel = paged_kernel(page_size=64, split=2)
    base_o, base_l = run(kernel, args)
    perm = torch.randperm(k_cache.shape[0], generator=torch.Generator().manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(len(perm))
    moved = [q, k_cache[perm], v_cache[perm], indptr, inv[indices.long()].to(torch.int32), last, scale]
    new_o, new_l = run(kernel, moved)
    assert np.array_equal(base_o, new_o) and np.array_equal(base_l, new_l)


@pytest.mark.parametrize("page_size", [1, 64])
def test_paged_decode_rising_maximum(page_size):
    """Scores that grow along a request's tokens: the softmax reference point of every row is raised
    several times inside a split or an item (the cold path: a rescale by a factor strictly between
    0 and 1), in the fixed-split, skewed, chunked and lockstep forms."""
    lens = [1500, 700, 65]
    args = C.paged_workload(lens, page_size=page_size, num_pages=4000 if page_size == 1 else 80, seed=3)
    q, k_cache, v_cache, indptr, indices = args[:5]
    q[..., 0] = 4.0
    d = q.shape[-1]
    for b, n in enumerate(lens):
        ramp = torch.linspace(0.0, 35.0 * d ** 0.5 / (4 * 1.4427), n).to(k_cache.dtype)
        pages = indices[int(indptr[b]):int(indptr[b + 1])].long()
        for i, pg in enumerate(pages.tolist()):
            chunk = ramp[i * page_size:(i + 1) * page_size]
            k_cache[pg, :len(chunk), :, 0] = chunk.reshape(-1, 1)
    if page_size == 1:
        args = args[:5] + args[6:]
    plans = [dict(split=None, waves=4), dict(split=4, waves=1), dict(split=8, waves=2, skew=30)]
    if page_size > 1:
        plans += [dict(split=8, waves=8, chunk_pages=4), dict(split=8, waves=8, chunk_pages=-1, lockstep=True)]
    for plan in plans:
        kernel = paged_kernel(page_size=page_size, **plan)
        print(f"paged rising maximum page={page_size} {plan}", flush=True)
        got_o, got_l = run(kernel, args)
        want_o, want_l = paged_oracle.decode(*args[:5], lens, page_size, args[-1], out_dtype="float16")
        np.testing.assert_allclose(got_o, want_o, rtol=1e-2, atol=1e-2)
        np.testing.assert_allclose(got_l, want_l, rtol=1e-3, atol=2e-3)


@pytest.mark.parametrize("d", [64, 256])
def test_paged_decode_other_head_widths(d):
    """64-wide heads (half a 128-feature block) and 256-wide ones (two blocks) through the single
    kernel, a fixed split and chunked items."""
    lens = [130, 9, 700, 0, 64]
    args = C.paged_workload(lens, page_size=16, num_pages=200, d=d)
    check(args, lens, 16, d=d, waves=2)
    check(args, lens, 16, d=d, waves=1, split=4)
    check(args, lens, 16, d=d, waves=8, split=8, chunk_pages=5, lockstep=True)
