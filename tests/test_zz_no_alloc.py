"""The fixed-scratch entry point of the C ABI (``chip_launch_seq_fixed_scratch``): a split
partial + combine pair launched with its partials inside the library's fixed per-GPU array and
caller-owned outputs, against the same pair launched through ``chip_launch_seq`` with the
partials in tensors.  Same kernels, same arithmetic order: the outputs must be bit-identical.
Two calls in a row, the second with a smaller input, so that the array's leftovers from the
first call lie where the second call's partials go."""

import ctypes

import numpy as np
import pytest
import torch

from cleave_amd import examples as C
from cleave_amd.codegen import HipCodeGen
from cleave_amd.dynamic.paging import (PAGED_DECODE_SLAB, CombineTiling, DenseAttention, PagingSpec,
                                       build_split_decode)
from cleave_amd.pipeline.direct import source_for
from cleave_amd.runtime import shim
from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code

pytestmark = pytest.mark.gpu


def _paged_pair(split=8, waves=4, chunk_pages=0):
    spec = PagingSpec(num_qo_heads=32, num_kv_heads=8, kind=PAGED_DECODE_SLAB, page_size=64)
    dense = DenseAttention(16, 32, 128, waves * 64, "float16", "float16", waves=waves, chunk_pages=chunk_pages)
    src = HipCodeGen().gen(build_split_decode(spec, dense, split, CombineTiling(split=split)))
    loaded = _load_main_kernel_from_code(src)
    return _compile(loaded, loaded.manifest["out_idx"]), _compile(loaded, None)


@pytest.mark.parametrize("chunk_pages", [0, 4])
def test_paged_decode_twice_second_call_smaller(chunk_pages):
    own, caller = _paged_pair(chunk_pages=chunk_pages)
    for lens in ([700, 64, 1500, 0, 333, 65, 2000, 1], [129, 40, 0]):      # the second call is the smaller one
        args = [a.cuda() if isinstance(a, torch.Tensor) else a for a in C.paged_workload(lens, page_size=64, num_pages=200)]
        want_o, want_l = own(*args)
        out = torch.full_like(want_o, float("nan"))
        lse = torch.full_like(want_l, float("nan"))
        print(f"fixed scratch: paged decode chunk_pages={chunk_pages} lens={lens}", flush=True)
        before = torch.cuda.memory_allocated()
        caller.call_fixed_scratch(*args, out, lse)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == before, "the fixed-scratch call allocated device memory through torch"
        assert torch.equal(out, want_o), "outputs differ from the chip_launch_seq path"
        assert np.array_equal(lse.cpu().numpy(), want_l.cpu().numpy())


def test_split_k_matmul_twice_second_call_smaller():
    for shapes in (dict(M=16, K=1024, N=768), dict(M=16, K=512, N=384)):
        prog = C.rmsnorm_matmul.trace(C.cl.f16, **shapes)
        src = source_for(prog, template="skinny", tiling=dict(WAVES_N=1, WAVES_K=2), split=4)
        loaded = _load_main_kernel_from_code(src)
        own, caller = _compile(loaded, loaded.manifest["out_idx"]), _compile(loaded, None)
        ins = [t.cuda() for t in C.inputs_c2(shapes)]
        want = own(*ins)
        out = torch.full_like(want, float("nan"))
        print(f"fixed scratch: rmsnorm matmul split-k=4 {shapes}", flush=True)
        caller.call_fixed_scratch(*ins, out, clear=True)         # (the clear is not needed by this kernel: exercised here)
        torch.cuda.synchronize()
        assert torch.equal(out, want)


def test_sizes_beyond_the_array_are_refused():
    own, caller = _paged_pair()
    args = [a.cuda() if isinstance(a, torch.Tensor) else a for a in C.paged_workload([64, 64], page_size=64, num_pages=8)]
    out, lse = own(*args)
    bound, dims, _ = caller._bind([*args, out, lse])
    fixed, nbytes = caller.fixed_scratch_layout(dims)
    assert 0 < nbytes <= shim.FIXED_SCRATCH_BYTES and all(off % 256 == 0 for off in fixed.values())
    descs, keep = caller._descs(bound, dims, fixed, [])
    with pytest.raises(shim.HipError, match="fixed array holds"):
        shim.launch_seq_fixed_scratch(descs, 0, [], shim.FIXED_SCRATCH_BYTES + 1)
    with pytest.raises(shim.HipError, match="multiple of 256"):
        shim.launch_seq_fixed_scratch(descs, 0, [(0, 0, 128)], 4096)
    with pytest.raises(shim.HipError, match="names no argument"):
        shim.launch_seq_fixed_scratch(descs, 0, [(len(descs), 0, 0)], 4096)
    with pytest.raises(shim.HipError, match="more than 64 scratch arguments"):
        shim.launch_seq_fixed_scratch(descs, 0, [(0, 0, 256 * i) for i in range(65)], 65 * 256)
    with pytest.raises(shim.HipError, match="named by two scratch entries"):
        shim.launch_seq_fixed_scratch(descs, 0, [(0, 0, 0), (0, 0, 256)], 4096)
    # (the refusals above come before anything is launched: the outputs of the last good call stand)
    torch.cuda.synchronize()
    again = own(*args)
    assert torch.equal(again[0], out) and torch.equal(again[1], lse)
    del keep
