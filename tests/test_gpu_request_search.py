"""GPU: the lane-parallel search of a row-pointer array that the chunked decode, the paged MLA
and the prefill kernels share (``cl_find_request`` in the common device header), against a plain
bisection on the host: request counts on both sides of the 64-lane and 256-entry boundaries,
empty requests (repeated pointers), pointers out of range (clamped), with and without the request
index in the key, the second pointer array."""

import numpy as np
import pytest
import torch

from cleave_amd.codegen import _template
from cleave_amd.runtime import shim

pytestmark = pytest.mark.gpu

KERNEL = r"""
extern "C" __global__ void __launch_bounds__(64)
probe(const int* __restrict__ ptr, const int* __restrict__ second, int batch, int limit, int limit2, int div, int with_b,
      const int* __restrict__ items, int* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const ClRequest r = cl_find_request(ptr, batch, limit, div, with_b, items[blockIdx.x], lane, second, limit2);
  if (lane == 0) {
    int* o = out + 5 * blockIdx.x;
    o[0] = r.req; o[1] = r.p0; o[2] = r.p1; o[3] = r.s0; o[4] = r.s1;
  }
}
"""


def _reference(ptr, second, batch, limit, limit2, div, with_b, item):
    clamp = lambda v, hi: min(max(int(v), 0), hi)                       # noqa: E731
    key = lambda b: with_b * b + clamp(ptr[b], limit) // div            # noqa: E731
    lo, hi = 0, batch - 1                                               # the last b with key(b) <= item (0 when none)
    while lo < hi:
        mid = (lo + hi + 1) // 2
        lo, hi = (mid, hi) if key(mid) <= item else (lo, mid - 1)
    return [lo, clamp(ptr[lo], limit), clamp(ptr[lo + 1], limit), clamp(second[lo], limit2), clamp(second[lo + 1], limit2)]


@pytest.mark.parametrize("batch", [1, 2, 5, 63, 64, 65, 200, 320, 321, 700])
def test_request_search_matches_bisection(batch):
    source = "#define CL_BF16 0\n" + _template("common.hip") + KERNEL
    code, _ = shim.compile_source(source, name="request_search.hip")
    mod = shim.Module(code)
    rng = np.random.default_rng(batch)
    for div, with_b in ((1, 0), (1, 1), (4, 1), (32, 1), (7, 1)):
        lens = rng.integers(0, 40, batch) * (rng.random(batch) < 0.8)   # a fifth of the requests are empty
        ptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        second = np.concatenate([[0], np.cumsum(rng.integers(0, 90, batch))]).astype(np.int32)
        limit, limit2 = int(ptr[-1]) - int(rng.integers(0, 3)), int(second[-1])      # now and then the tail is clamped
        limit = max(limit, 1)
        top = with_b * batch + limit // div + 3
        items = rng.integers(0, top, 300).astype(np.int32)
        d_ptr, d_second, d_items = (torch.from_numpy(a).cuda() for a in (ptr, second, items))
        out = torch.full((len(items), 5), -7, dtype=torch.int32, device="cuda")
        args = shim.PackedArgs([("ptr", d_ptr.data_ptr()), ("ptr", d_second.data_ptr()), ("i32", batch), ("i32", limit),
                                ("i32", limit2), ("i32", div), ("i32", with_b), ("ptr", d_items.data_ptr()),
                                ("ptr", out.data_ptr())])
        print(f"request search batch={batch} div={div} with_b={with_b} limit={limit}", flush=True)
        shim.launch_seq([shim.make_desc(mod.function("probe"), (len(items), 1, 1), (64, 1, 1), 0, args)],
                        torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want = np.array([_reference(ptr, second, batch, limit, limit2, div, with_b, int(t)) for t in items])
        np.testing.assert_array_equal(out.cpu().numpy(), want)
