"""Paged GQA decode out of a 300 000-page pool: the property that defines the paged benchmark
configuration.

A page is 64 x 8 x 128 f16 = 131 072 bytes, so byte offsets pass 2^31 from page 16 384 on and 2^32
from page 32 768 on; the two pools are 39.3 GB each.  They are allocated without being filled; only
the pages a seeded table names are written.  The table is drawn from a seeded permutation of the
whole pool and forced to contain page 0, the pages either side of the 2^31 and 2^32 byte
boundaries, and the last page.  Checks, for the chunked plan the benchmark selects, the unlimited
chunk and a fixed-split plan:

  * the gather is bit-exact: saturating one-hot queries turn the output into one gathered V row
    whose bits encode (page, slot, head) -- a page id truncated to 32-bit byte offsets, a wrong
    slot or a wrong head changes bits;
  * the attention output equals the numpy oracle's on the named pages compacted into a small pool
    (reference ``python/cleave/dynamic/reference.py:143-200``), rtol = atol = 1e-2, lse 1e-3;
  * the same comparison at the request lengths the configuration states: 32 requests with lengths
    drawn uniformly from [256, 16384] (up to 256 pages a request, several thousand pages in all),
    placed at seeded ids across the whole pool.
"""

import numpy as np
import pytest
import torch

from oracle import paged_oracle
from tests.test_gpu_paged import paged_kernel

pytestmark = pytest.mark.gpu

POOL, PAGE, HKV, HQ, D = 300_000, 64, 8, 32, 128
LENS = [257, 64 * 9, 1, 64 * 17 + 5, 0, 1999, 640, 64 * 30 + 63]
FORCED = [0, 16_383, 16_384, 16_385, 32_767, 32_768, 32_769, 65_536, 131_072, 262_144, POOL - 2, POOL - 1]
PLANS = [dict(split=8, waves=8, chunk_pages=16), dict(split=8, waves=8, chunk_pages=-1, lockstep=True), dict(split=8, waves=4),
         dict(split=8, waves=1, skew=30)]


def _table(seed=21):
    gen = torch.Generator(device="cpu").manual_seed(seed)
    pages = [-(-n // PAGE) for n in LENS]
    total = sum(pages)
    drawn = [p for p in torch.randperm(POOL, generator=gen).tolist() if p not in FORCED][:total - len(FORCED)]
    ids = torch.tensor(FORCED + drawn)[torch.randperm(total, generator=gen)]
    indptr = torch.tensor([0] + np.cumsum(pages).tolist(), dtype=torch.int32)
    last = torch.tensor([n - (p - 1) * PAGE if p else 0 for n, p in zip(LENS, pages)], dtype=torch.int32)
    return gen, ids.to(torch.int32), indptr, last


@pytest.fixture(scope="module")
def pools():
    need = 2 * POOL * PAGE * HKV * D * 2
    free, _ = torch.cuda.mem_get_info()
    if free < need + (8 << 30):
        pytest.skip(f"needs {need / 2**30:.0f} GiB of free device memory for the two pools, {free / 2**30:.0f} free")
    print(f"allocating two pools of {POOL} pages ({need / 2**30:.1f} GiB)", flush=True)
    k = torch.empty((POOL, PAGE, HKV, D), dtype=torch.float16, device="cuda")
    v = torch.empty((POOL, PAGE, HKV, D), dtype=torch.float16, device="cuda")
    yield k, v
    del k, v
    torch.cuda.empty_cache()


def _run(kernel, args):
    out, lse = kernel(*args)
    torch.cuda.synchronize()
    return out.float().cpu().numpy(), lse.cpu().numpy()


@pytest.mark.parametrize("plan", PLANS, ids=lambda p: "-".join(f"{k}{v}" for k, v in p.items()))
def test_attention_over_high_pages_matches_the_oracle(pools, plan):
    k_pool, v_pool = pools
    gen, ids, indptr, last = _table()
    assert int(ids.max()) == POOL - 1 and int((ids >= 16_384).sum()) > 8
    n = len(ids)
    k_small = torch.randn(n, PAGE, HKV, D, generator=gen).to(torch.float16)
    v_small = torch.randn(n, PAGE, HKV, D, generator=gen).to(torch.float16)
    q = torch.randn(len(LENS), HQ, D, generator=gen).to(torch.float16)
    k_pool[ids.long().cuda()] = k_small.cuda()
    v_pool[ids.long().cuda()] = v_small.cuda()
    scale = D ** -0.5
    print(f"pool300k attention plan={plan}", flush=True)
    kernel = paged_kernel(page_size=PAGE, **plan)
    got_o, got_l = _run(kernel, [q.cuda(), k_pool, v_pool, indptr.cuda(), ids.cuda(), last.cuda(), scale])
    # the oracle sees the same pages compacted: table entry i names small-pool page i
    want_o, want_l = paged_oracle.decode(q, k_small, v_small, indptr, torch.arange(n, dtype=torch.int32), LENS, PAGE,
                                         scale, out_dtype="float16")
    np.testing.assert_allclose(got_o, want_o, rtol=1e-2, atol=1e-2)
    live = np.isfinite(want_l)
    np.testing.assert_allclose(got_l[live], want_l[live], rtol=1e-3, atol=1e-3)
    assert np.all(np.isneginf(got_l[~live])) and np.all(got_o[np.array(LENS) == 0] == 0)


@pytest.mark.parametrize("plan", PLANS, ids=lambda p: "-".join(f"{k}{v}" for k, v in p.items()))
def test_gather_out_of_high_pages_is_bit_exact(pools, plan):
    """Every request's query saturates the softmax on one token; the tokens are chosen so that the
    forced pages (first, last, both sides of 2^31 and 2^32 bytes) are among the gathered ones."""
    k_pool, v_pool = pools
    gen, ids, indptr, last = _table()
    n = len(ids)
    where = {int(p): i for i, p in enumerate(ids.tolist())}
    ptr = indptr.tolist()
    live = [b for b, ln in enumerate(LENS) if ln]
    # V rows carry (table position, slot, head) in their bits; K is zero but for the target tokens
    code = torch.arange(n * PAGE * HKV).reshape(n, PAGE, HKV)
    v_small = ((code % 2039).to(torch.float16) / 8.0)[..., None].expand(-1, -1, -1, D).contiguous()
    forced_in = {b: [where[p] for p in FORCED if ptr[b] <= where[p] < ptr[b + 1]] for b in live}
    tested = set()
    for rnd in range(max(2, max(len(f) for f in forced_in.values()))):
        k_small = torch.zeros(n, PAGE, HKV, D, dtype=torch.float16)
        targets = {}
        for b in live:
            first, stop = ptr[b], ptr[b + 1]
            # prefer a forced page inside this request's slice of the table, a different one per round
            forced_here = forced_in[b]
            pos = forced_here[rnd % len(forced_here)] if forced_here else first + (7 * b + 3 * rnd) % (stop - first)
            tested.add(int(ids[pos]))
            slot_limit = PAGE if pos < stop - 1 else int(last[b])
            slot = (11 * b + 5 * rnd) % slot_limit
            k_small[pos, slot, :, 3] = 60.0
            targets[b] = (pos, slot)
        q = torch.zeros(len(LENS), HQ, D, dtype=torch.float16)
        q[:, :, 3] = 60.0
        k_pool[ids.long().cuda()] = k_small.cuda()
        v_pool[ids.long().cuda()] = v_small.cuda()
        print(f"pool300k one-hot gather plan={plan} round={rnd} pages={[int(ids[p]) for p, _ in targets.values()]}",
              flush=True)
        kernel = paged_kernel(page_size=PAGE, **plan)
        got_o, _ = _run(kernel, [q.cuda(), k_pool, v_pool, indptr.cuda(), ids.cuda(), last.cuda(), 1.0])
        for b, (pos, slot) in targets.items():
            for h in range(HQ):
                want = v_small[pos, slot, h // (HQ // HKV)].float().numpy()
                assert np.array_equal(got_o[b, h], want), (b, h, int(ids[pos]), slot)
    assert set(FORCED) <= tested


def _stated_draw(seed=5):
    """The benchmark's own draw (bench.py ``run_paged``): 32 lengths U[256, 16384] from the seed, the table a
    seeded permutation of the whole pool (``python/cleave/dynamic/reference.py:44-49``), with the pool's last
    page put in so that the highest address is among the ones read."""
    gen = torch.Generator(device="cpu").manual_seed(seed)
    lens = torch.randint(256, 16384 + 1, (32,), generator=gen).tolist()
    pages = [-(-n // PAGE) for n in lens]
    total = sum(pages)
    ids = torch.randperm(POOL, generator=gen)[:total]
    if POOL - 1 not in ids.tolist():
        ids[total // 2] = POOL - 1
    indptr = torch.tensor([0] + np.cumsum(pages).tolist(), dtype=torch.int32)
    last = torch.tensor([n - (p - 1) * PAGE for n, p in zip(lens, pages)], dtype=torch.int32)
    return gen, lens, ids.to(torch.int32), indptr, last


@pytest.fixture(scope="module")
def stated():
    """The draw, its operands and the oracle's answer, made once for the three plans (the oracle takes ~12 s)."""
    gen, lens, ids, indptr, last = _stated_draw()
    n = len(ids)
    k_small = torch.randn(n, PAGE, HKV, D, generator=gen).to(torch.float16)
    v_small = torch.randn(n, PAGE, HKV, D, generator=gen).to(torch.float16)
    q = torch.randn(len(lens), HQ, D, generator=gen).to(torch.float16)
    want = paged_oracle.decode(q, k_small, v_small, indptr, torch.arange(n, dtype=torch.int32), lens, PAGE, D ** -0.5,
                               out_dtype="float16")
    return lens, ids, indptr, last, q, k_small, v_small, want


@pytest.mark.parametrize("plan", PLANS, ids=lambda p: "-".join(f"{k}{v}" for k, v in p.items()))
def test_the_stated_request_lengths_match_the_oracle(pools, stated, plan):
    k_pool, v_pool = pools
    lens, ids, indptr, last, q, k_small, v_small, (want_o, want_l) = stated
    n = len(ids)
    assert min(lens) >= 256 and max(lens) > 12_000 and int((indptr[1:] - indptr[:-1]).max()) > 190 and n > 3000
    assert int(ids.max()) == POOL - 1 and int((ids >= 16_384).sum()) > 0.9 * n and len(set(ids.tolist())) == n
    k_pool[ids.long().cuda()] = k_small.cuda()
    v_pool[ids.long().cuda()] = v_small.cuda()
    print(f"pool300k stated lengths plan={plan}: {sum(lens)} tokens in {n} pages, longest {max(lens)}", flush=True)
    kernel = paged_kernel(page_size=PAGE, **plan)
    got_o, got_l = _run(kernel, [q.cuda(), k_pool, v_pool, indptr.cuda(), ids.cuda(), last.cuda(), D ** -0.5])
    np.testing.assert_allclose(got_o, want_o, rtol=1e-2, atol=1e-2)
    np.testing.assert_allclose(got_l, want_l, rtol=1e-3, atol=1e-3)
