"""GPU parity of the SwiGLU operator ``(x @ w_up) * silu(x @ w_gate)`` (the reference's
``demo/swiglu.py``; graph ``tests/_graphs.py:403-436``) against the numpy oracle: explicit
tilings of the two-halved B tile (both weight layouts, both element types, ragged edges), the
searched candidates end to end through ``compile``, and the benchmark size checked on a sample of
rows and columns."""

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


@cleave_amd.jit
def swiglu_nk(x: cl.Tensor["M", "K"], w_up: cl.Tensor["N", "K"], w_gate: cl.Tensor["N", "K"]):
    return (x @ w_up.mT) * cl.silu(x @ w_gate.mT)


def _inputs(prog, seed):
    x, wu, wg = prog.random_inputs(seed=seed)
    k = x.shape[-1]
    return x, (wu.float() / k ** 0.5).to(wu.dtype), (wg.float() / k ** 0.5).to(wg.dtype)


def _check(fn, dtype, shapes, tiling, seed=3):
    prog = fn.trace(dtype, **shapes)
    args = _inputs(prog, seed)
    print(f"swiglu case {prog.name} {dtype} {shapes} {tiling}", flush=True)
    out = kernel_for(prog, template="gemm_dma", tiling=dict(tiling, BK=64, SWIGLU=1))(*args)
    torch.cuda.synchronize()
    want = program_oracle.evaluate(prog, list(args))[0]
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)


TILINGS = [dict(BM=64, BN=64, WM=2, WN=1), dict(BM=128, BN=128, WM=2, WN=2), dict(BM=256, BN=256, WM=4, WN=2),
           dict(BM=32, BN=128, WM=1, WN=4), dict(BM=128, BN=256, WM=2, WN=4)]


@pytest.mark.parametrize("tiling", TILINGS, ids=lambda t: f"{t['BM']}x{t['BN']}_{t['WM']}x{t['WN']}")
@pytest.mark.parametrize("fn", [C.swiglu, swiglu_nk], ids=["w_kn", "w_nk"])
def test_swiglu_tilings(fn, tiling):
    _check(fn, cl.f16, dict(M=256, N=512, K=256), tiling)


def test_swiglu_bf16_and_ragged_rows():
    _check(C.swiglu, cl.bf16, dict(M=200, N=384, K=192), dict(BM=64, BN=256, WM=2, WN=2))
    _check(swiglu_nk, cl.bf16, dict(M=72, N=128, K=64), dict(BM=64, BN=128, WM=1, WN=2))


def test_swiglu_compiles_end_to_end(cache_root):
    shapes = dict(M=512, N=1024, K=512)
    kernel = P.compile(C.swiglu, shapes=shapes, dtype=cl.f16, split=False, schedule=P.ScheduleConfig(topk=4),
                       eval=P.EvalConfig(warmup=2, iters=10, max_parallel=2))
    rep = kernel.report
    assert kernel.variant == "solo" and len(rep.correct) == len(rep) >= 1
    prog = cleave_amd.trace(C.swiglu, shapes, cl.f16)
    args = _inputs(prog, 5)
    want = program_oracle.evaluate(prog, list(args))[0]
    np.testing.assert_allclose(kernel(*args).float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)


def test_swiglu_benchmark_size_on_a_sample():
    """4096 x 14336 x 4096: the searched best tiling, checked on 48 rows x 320 columns spread over
    the output (the oracle on the whole of it would take minutes)."""
    shapes = C.FULL["swiglu"]
    prog = C.swiglu.trace(cl.f16, **shapes)
    x, wu, wg = _inputs(prog, 11)
    out = kernel_for(prog)(x, wu, wg)
    torch.cuda.synchronize()
    gen = np.random.default_rng(0)
    rows = np.sort(gen.choice(shapes["M"], 48, replace=False))
    cols = np.sort(gen.choice(shapes["N"], 320, replace=False))
    xs = x[torch.from_numpy(rows).cuda()].float().cpu().numpy()
    up = xs @ wu[:, torch.from_numpy(cols).cuda()].float().cpu().numpy()
    gate = xs @ wg[:, torch.from_numpy(cols).cuda()].float().cpu().numpy()
    want = up * (gate / (1.0 + np.exp(-gate)))
    got = out[torch.from_numpy(rows).cuda()][:, torch.from_numpy(cols).cuda()].float().cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=1e-2, atol=1e-2)
