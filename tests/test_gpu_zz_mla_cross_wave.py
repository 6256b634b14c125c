"""GPU parity cases of the cross-wave MLA decode kernel (tiling XW=1) against the numpy oracle.

The kernel is withdrawn: its split form once returned a wrong result (20 372 of 32 768 elements, late
in a long session, never alone), reading the flag / candidate / reference handshake and the load
accounting found no cause, and it measured no faster than the one-wave-per-head-set kernel.  The code
generator now refuses XW=1, so these cases are skipped; they stay as the cases to run should the kernel
ever come back with the cause known."""

import numpy as np
import pytest
import torch

from oracle import program_oracle as po
from cleave_amd import examples as C
from cleave_amd.pipeline.direct import kernel_for
from tests.test_gpu_kernels import ATOL, RTOL, _check

pytestmark = [pytest.mark.gpu,
              pytest.mark.skip(reason="cross-wave MLA decode kernel withdrawn: one unexplained wrong result of its "
                                      "split form; the code generator refuses tiling XW=1")]


def test_mla_decode_cross_wave_small():
    """64 heads per workgroup, scores and values shared out over the waves two ways: a ragged kv
    length (masked tail, clamped loads), more than one head group, splits one step long, and a
    split count that leaves the last split without any step."""
    fn, dt, mk = C.CASES["c4"]
    for shapes, splits in ((dict(B=2, H=64, D=512, PE=64, SKV=160), (None, 2, 5)),
                           (dict(B=1, H=128, D=256, PE=64, SKV=77), (None, 7)),
                           (dict(B=3, H=64, D=512, PE=64, SKV=32), (None, 2))):
        for split in splits:
            _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(XW=1), split=split)


def test_mla_decode_cross_wave_rising_maximum():
    """Scores that keep growing along the KV axis: the workgroup-wide raise of the softmax
    reference (flag beside the weights, rescale of every wave's accumulators, weights redone
    from the kept scores) is taken several times per split and must stay exact."""
    fn, dt, mk = C.CASES["c4"]
    shapes = dict(B=1, H=64, D=512, PE=64, SKV=512)
    prog = fn.trace(dt, **shapes)
    q, kv, q_pe, k_pe = mk(shapes, device="cpu")
    ramp = torch.linspace(0.2, 6.0, shapes["SKV"]).reshape(1, -1, 1)
    kv = (kv.float() * 0.2 + ramp * torch.sign(q.float().mean(dim=(1,), keepdim=True))).to(kv.dtype)
    ins = [q, kv, q_pe, k_pe]
    want = po.evaluate(prog, ins)[0]
    for split in (None, 2):
        kernel = kernel_for(prog, template="mla_decode", tiling=dict(XW=1), split=split)
        print(f"case mla cross-wave rising maximum split={split}", flush=True)
        got = kernel(*[t.cuda() for t in ins]).float().cpu().numpy().reshape(want.shape)
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("split", [8, 16])
def test_mla_decode_cross_wave_c4_full(split):
    fn, dt, mk = C.CASES["c4"]
    _check(fn.trace(dt, **C.FULL["c4"]), mk, C.FULL["c4"], template="mla_decode", tiling=dict(XW=1), split=split)
