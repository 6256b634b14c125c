"""GPU parity of LoRA ``x @ w + (x @ a) @ b`` (the reference's ``demo/lora.py``; graph
``tests/_graphs.py:438-480``) against the numpy oracle: every shape of the few-row kernel's wave
grid, ranks 8 / 16 / 32, ragged rows and column slabs, both element types, the benchmark size,
and ``compile`` end to end."""

import numpy as np
import pytest
import torch

import cleave_amd
import cleave_amd.lang as cl
from cleave_amd import pipeline as P
from oracle import program_oracle
from cleave_amd import examples as C
from cleave_amd.pipeline.direct import kernel_for

pytestmark = pytest.mark.gpu


def _inputs(prog, seed):
    x, w, a, b = prog.random_inputs(seed=seed)
    k, r = x.shape[-1], a.shape[-1]
    scale = lambda t, n: (t.float() / n ** 0.5).to(t.dtype)   # noqa: E731
    return x, scale(w, k), scale(a, k), scale(b, r)


def _check(dtype, shapes, tiling=None, seed=5):
    prog = C.lora.trace(dtype, **shapes)
    args = _inputs(prog, seed)
    print(f"lora case {dtype} {shapes} {tiling}", flush=True)
    k = kernel_for(prog, template="skinny", tiling=dict(tiling, LORA=1)) if tiling else kernel_for(prog)
    out = k(*args)
    torch.cuda.synchronize()
    want = program_oracle.evaluate(prog, list(args))[0]
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("tiling", [dict(WAVES_N=1, WAVES_K=1), dict(WAVES_N=1, WAVES_K=4), dict(WAVES_N=2, WAVES_K=2),
                                    dict(WAVES_N=1, WAVES_K=8, PREFETCH=1), dict(WAVES_N=4, WAVES_K=1)],
                         ids=lambda t: f"n{t['WAVES_N']}k{t['WAVES_K']}")
def test_lora_wave_grids(tiling):
    _check(cl.f16, dict(M=16, N=512, K=512, R=16), tiling)
    if tiling["WAVES_K"] < 8:     # (three row tiles times eight K-sharing waves would not fit the reduction into LDS)
        _check(cl.f16, dict(M=40, N=328, K=288, R=8), tiling)      # ragged rows and last column slab, 9 steps
    else:
        _check(cl.f16, dict(M=9, N=328, K=288, R=8), tiling)


def test_lora_ranks_types_and_benchmark_size():
    _check(cl.bf16, dict(M=16, N=256, K=256, R=32), dict(WAVES_N=1, WAVES_K=2))
    _check(cl.f16, dict(M=64, N=256, K=128, R=64), dict(WAVES_N=1, WAVES_K=2))
    _check(cl.f16, C.FULL["lora"])


@pytest.mark.parametrize("split,tiling", [(2, dict(WAVES_N=1, WAVES_K=1)), (4, dict(WAVES_N=1, WAVES_K=2)),
                                          (8, dict(WAVES_N=2, WAVES_K=2))], ids=["s2", "s4", "s8"])
def test_lora_split_over_k(split, tiling):
    """Partial sums of both products per K split; the combine adds them up and applies the rank update."""
    for dtype, shapes in ((cl.f16, dict(M=16, N=512, K=1024, R=16)), (cl.bf16, dict(M=40, N=256, K=512, R=32))):
        prog = C.lora.trace(dtype, **shapes)
        args = _inputs(prog, 8)
        print(f"lora split case {dtype} {shapes} split={split} {tiling}", flush=True)
        out = kernel_for(prog, template="skinny", tiling=dict(tiling, LORA=1), split=split)(*args)
        torch.cuda.synchronize()
        np.testing.assert_allclose(out.float().cpu().numpy(), program_oracle.evaluate(prog, list(args))[0],
                                   rtol=1e-2, atol=1e-2)


def test_lora_benchmark_size_picks_a_split_variant(cache_root):
    kernel = P.compile(C.lora, shapes=C.FULL["lora"], dtype=cl.f16, split=cl.Split("K", (4, 8)),
                       schedule=P.ScheduleConfig(topk=3, split_k=(4, 8)), eval=P.EvalConfig(warmup=2, iters=20, max_parallel=2))
    rep = kernel.report
    assert len(rep.correct) == len(rep) and kernel.variant.startswith("split")
    prog = cleave_amd.trace(C.lora, C.FULL["lora"], cl.f16)
    args = _inputs(prog, 10)
    np.testing.assert_allclose(kernel(*args).float().cpu().numpy(), program_oracle.evaluate(prog, list(args))[0],
                               rtol=1e-2, atol=1e-2)


def test_lora_compiles_end_to_end(cache_root):
    shapes = dict(M=16, N=1024, K=1024, R=16)
    kernel = P.compile(C.lora, shapes=shapes, dtype=cl.f16, split=False, schedule=P.ScheduleConfig(topk=4),
                       eval=P.EvalConfig(warmup=2, iters=10, max_parallel=2))
    assert kernel.variant == "solo" and len(kernel.report.correct) == len(kernel.report) >= 1
    prog = cleave_amd.trace(C.lora, shapes, cl.f16)
    args = _inputs(prog, 6)
    np.testing.assert_allclose(kernel(*args).float().cpu().numpy(), program_oracle.evaluate(prog, list(args))[0],
                               rtol=1e-2, atol=1e-2)
