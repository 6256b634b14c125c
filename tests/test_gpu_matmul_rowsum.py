"""GPU parity of matmul + row sum ``(x @ w).sum(-1)`` (the reference's ``tests/_graphs.py:150-160``)
against the numpy oracle: explicit tilings of the column-walking kernel (both weight layouts, odd
and even numbers of steps, ragged rows), the searched best at the benchmark size, and ``compile``
end to end."""

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
def matmul_rowsum_nk(x: cl.Tensor["M", "K"], w: cl.Tensor["N", "K"]):
    return (x @ w.mT).sum(dim=-1, keepdim=True)


def _inputs(prog, seed):
    x, w = prog.random_inputs(seed=seed)
    return x, (w.float() / x.shape[-1] ** 0.5).to(w.dtype)


def _check(fn, dtype, shapes, tiling=None, seed=4):
    prog = fn.trace(dtype, **shapes)
    args = _inputs(prog, seed)
    print(f"matmul_rowsum case {prog.name} {dtype} {shapes} {tiling}", flush=True)
    k = kernel_for(prog, template="gemm_dma", tiling=dict(tiling, BK=64, ROWSUM=1)) if tiling else kernel_for(prog)
    out = k(*args)
    torch.cuda.synchronize()
    want = program_oracle.evaluate(prog, list(args))[0]
    # a row sums N products of O(1): the tolerance scales with the sum's own rounding grid
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2 * max(1.0, np.abs(want).max() / 8))


@pytest.mark.parametrize("tiling", [dict(BM=16, BN=256, WM=1, WN=4), dict(BM=64, BN=128, WM=2, WN=2),
                                    dict(BM=128, BN=64, WM=4, WN=1), dict(BM=32, BN=256, WM=2, WN=4)],
                         ids=lambda t: f"{t['BM']}x{t['BN']}_{t['WM']}x{t['WN']}")
@pytest.mark.parametrize("fn", [C.matmul_rowsum, matmul_rowsum_nk], ids=["w_kn", "w_nk"])
def test_matmul_rowsum_tilings(fn, tiling):
    _check(fn, cl.f16, dict(M=256, N=768, K=64), tiling)       # 3, 6 or 12 steps
    _check(fn, cl.f16, dict(M=200, N=512, K=192), tiling)      # ragged rows, several K steps per column tile


def test_matmul_rowsum_bf16_and_benchmark_size():
    _check(C.matmul_rowsum, cl.bf16, dict(M=128, N=256, K=128), dict(BM=16, BN=256, WM=1, WN=4))
    _check(C.matmul_rowsum, cl.f16, C.FULL["matmul_rowsum"])


def test_matmul_rowsum_compiles_end_to_end(cache_root):
    shapes = dict(M=512, N=1024, K=128)
    kernel = P.compile(C.matmul_rowsum, shapes=shapes, dtype=cl.f16, split=False, schedule=P.ScheduleConfig(topk=4),
                       eval=P.EvalConfig(warmup=2, iters=10, max_parallel=2))
    assert kernel.variant == "solo" and len(kernel.report.correct) == len(kernel.report) >= 1
    prog = cleave_amd.trace(C.matmul_rowsum, shapes, cl.f16)
    args = _inputs(prog, 9)
    want = program_oracle.evaluate(prog, list(args))[0]
    np.testing.assert_allclose(kernel(*args).float().cpu().numpy(), want, rtol=1e-2, atol=2e-2)
