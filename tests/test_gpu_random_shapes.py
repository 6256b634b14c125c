"""Seeded draws of shapes, templates, tilings and split factors for the dense kernel families,
each checked against the numpy oracle at rtol = atol = 1e-2: a net for edge handling (ragged rows,
columns and key counts, odd step counts, splits with empty or one-step ranges, every wave grid the
search may propose) beside the hand-picked cases of the other files.  A drawn combination that the
lowering or the emitter refuses (a split that does not divide its extent, an LDS budget) counts
as drawn, not as passed: at least two thirds of every seed's draws must run."""

import random

import numpy as np
import pytest

import cleave_amd.lang as cl
from cleave_amd import examples as C
from cleave_amd.core.errors import CleaveError
from cleave_amd.lower.stages import split_stages
from cleave_amd.pipeline.direct import kernel_for, stage_graph
from cleave_amd.schedule import search_tiling
from oracle import program_oracle as po

pytestmark = pytest.mark.gpu
DRAWS = 36
PAGED_DRAWS = 24


def _draw(rng, n):
    """(label, program, inputs, kernel_for keywords) of one draw."""
    family = rng.choice(["matmul", "matmul", "few rows", "decode", "many rows", "mla"])
    if family == "matmul":
        shapes = dict(M=rng.randrange(1, 700), N=8 * rng.randrange(1, 100), K=64 * rng.randrange(1, 12))
        program, inputs = C.matmul.trace(cl.f16, **shapes), C.inputs_c1(shapes, seed=n)
        split = rng.choice([None, None, 2, 3])
        if split and (shapes["K"] // 64) % split:
            split = None
        graph = stage_graph(program)
        pick = rng.choice(search_tiling(split_stages(graph, split)[0] if split else graph, topk=400))
        return f"matmul {shapes}", program, inputs, dict(template=pick.template, tiling=dict(pick.tiling), split=split)
    if family == "few rows":
        shapes = dict(M=rng.randrange(1, 65), N=8 * rng.randrange(1, 300), K=32 * rng.randrange(1, 64))
        split = rng.choice([None, 2, 4, 8])
        if split and (shapes["K"] // 32) % split:
            split = None
        tiling = dict(WAVES_N=rng.choice([1, 2]), WAVES_K=rng.choice([1, 2, 4]), PREFETCH=rng.choice([1, 2, 3]))
        return (f"rmsnorm_matmul {shapes}", C.rmsnorm_matmul.trace(cl.f16, **shapes), C.inputs_c2(shapes, seed=n),
                dict(template="skinny", tiling=tiling, split=split))
    if family in ("decode", "many rows"):
        kv_heads, group = rng.choice([1, 2, 4]), rng.choice([1, 2, 4, 8])
        decode = family == "decode"
        shapes = dict(HQ=kv_heads * group, HKV=kv_heads, SQ=rng.choice([1, 1, 2, 3]) if decode else rng.randrange(64, 300),
                      SKV=rng.randrange(1, 700), D=rng.choice([64, 128] if decode else [64, 128, 256]))
        split = rng.choice([None, 2, 4, 8] if decode else [None, None, 2, 4])
        if split:
            shapes["SKV"] = max(split, shapes["SKV"] - shapes["SKV"] % split)
        how = (dict(template="attn_decode", tiling=dict(WAVES=rng.choice([1, 2, 4, 8]), PREFETCH=rng.choice([1, 2]))) if decode
               else dict(template="attn_prefill", tiling=dict(SHARED=1)))
        return (f"attention {shapes}", C.gqa_decode_exact.trace(cl.f16, **shapes), C.inputs_c3(shapes, seed=n),
                dict(how, split=split))
    shapes = dict(B=rng.randrange(1, 4), H=rng.choice([64, 128]), D=rng.choice([256, 512]), PE=64, SKV=rng.randrange(1, 500))
    split = rng.choice([None, 2, 4, 8])
    if split:
        shapes["SKV"] = max(split, shapes["SKV"] - shapes["SKV"] % split)
    panels = (shapes["D"] + 64) // 64
    tiling = rng.choice([dict(DUO=1), dict(DUO=1, LDS_AHEAD=4, S_PANELS=rng.randrange(1, panels)), dict(WAVES=4, HG=1),
                         dict(DUO=1, LDS_AHEAD=2)])
    return (f"mla_decode {shapes}", C.mla_decode.trace(cl.bf16, **shapes), C.inputs_c4(shapes, seed=n),
            dict(template="mla_decode", tiling=tiling, split=split))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_drawn_shapes_and_tilings_against_the_oracle(seed):
    rng = random.Random(seed)
    ran = 0
    for n in range(DRAWS):
        label, program, inputs, how = _draw(rng, 1000 * seed + n)
        print(f"case drawn {label} {how}", flush=True)
        try:
            kernel = kernel_for(program, **how)
        except CleaveError as refusal:
            print(f"    refused: {str(refusal)[:120]}", flush=True)
            continue
        got = kernel(*[t.cuda() for t in inputs]).float().cpu().numpy()
        want = po.evaluate(program, inputs)[0]
        np.testing.assert_allclose(got.reshape(want.shape), want, rtol=1e-2, atol=1e-2, err_msg=f"{label} {how}")
        ran += 1
    assert 3 * ran >= 2 * DRAWS, f"only {ran} of {DRAWS} draws ran"


@pytest.mark.parametrize("seed", [21, 22])
def test_drawn_paged_decode_requests_against_the_oracle(seed):
    """Paged decode over drawn page sizes, head groups, request lengths (empty, one token, under a
    page, many pages), wave counts, splits and chunked work items; the log-sum-exp row of an empty
    request is -inf and its output row zero."""
    from tests.test_gpu_paged import check
    rng = random.Random(seed)
    for n in range(PAGED_DRAWS):
        page = rng.choice([1, 16, 64])
        kv_heads, group = rng.choice([2, 4, 8]), rng.choice([2, 4, 8])
        if kv_heads * group > 32:
            kv_heads = 32 // group
        lens = [rng.choice([0, 1, rng.randrange(1, 70), rng.randrange(1, 2000)]) for _ in range(rng.randrange(1, 12))]
        pages = sum(-(-length // page) for length in lens) + rng.randrange(1, 50)
        args = C.paged_workload(lens, page_size=page, num_pages=pages, hq=kv_heads * group, hkv=kv_heads, seed=1000 * seed + n)
        if page == 1:
            args = args[:5] + args[6:]
        how = dict(waves=rng.choice([1, 2, 4, 8]), split=rng.choice([None, 2, 4, 8]), hq=kv_heads * group, hkv=kv_heads)
        if how["split"] and page == 64 and rng.random() < 0.5:
            how.update(chunk_pages=rng.choice([1, 3, 16, -1]), prefetch=rng.choice([1, 2]), waves=8,
                       lockstep=rng.choice([False, True]))
        check(args, lens, page, **how)
