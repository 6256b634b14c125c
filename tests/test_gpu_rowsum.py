"""GPU parity of the row reductions ``x.sum(-1)`` and ``x / x.sum(-1)`` (the reference's ``rowsum``
and ``rowsum_div`` cases, ``tests/_graphs.py:1238-1275``) against the numpy oracle: every
rows-per-workgroup shape, row lengths around the 512-element chunk and the four-chunk trip,
ragged row counts, both element types, the reference's size, ``compile`` end to end."""

import numpy as np
import pytest
import torch

import cleave_amd.lang as cl
from cleave_amd import pipeline as P
from oracle import program_oracle
from cleave_amd import examples as C
from cleave_amd.pipeline.direct import kernel_for

pytestmark = pytest.mark.gpu


def _check(fn, dtype, shapes, rows=None, seed=3):
    prog = fn.trace(dtype, **shapes)
    (x,) = prog.random_inputs(seed=seed)
    x = (x.float().abs() + 0.25).to(x.dtype)                 # positive entries: the divisor stays away from 0
    print(f"row reduction case {prog.name} {dtype} {shapes} rows/block={rows}", flush=True)
    k = kernel_for(prog, template="rowsum", tiling=dict(ROWS_PER_BLOCK=rows)) if rows else kernel_for(prog)
    out = k(x)
    torch.cuda.synchronize()
    want = program_oracle.evaluate(prog, [x])[0]
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("rows", [1, 2, 4])
@pytest.mark.parametrize("fn", [C.rowsum, C.rowsum_div], ids=["sum", "div"])
def test_row_reductions(fn, rows):
    for n in (8, 504, 512, 520, 2048, 2056, 4104, 8192, 8704):     # (whole 512-element pieces up to 8192 stay in registers)
        _check(fn, cl.f16, dict(M=37, N=n), rows)


def test_row_reductions_bf16_reference_size_and_compile(cache_root):
    _check(C.rowsum_div, cl.bf16, dict(M=130, N=1000))
    _check(C.rowsum, cl.f16, dict(M=4096, N=4096))
    _check(C.rowsum_div, cl.f16, dict(M=4096, N=4096))
    kernel = P.compile(C.rowsum_div, shapes=dict(M=256, N=1024), dtype=cl.f16, split=False,
                       schedule=P.ScheduleConfig(topk=3), eval=P.EvalConfig(warmup=2, iters=10, max_parallel=2))
    assert len(kernel.report.correct) == len(kernel.report) == 3
