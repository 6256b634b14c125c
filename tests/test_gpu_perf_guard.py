"""Latency of fixed plans against this GPU model's recorded figures
(``tests/golden/perf_mi355x.json``): the plans ``bench.py`` selects for the graded operators, built
without a search, their dominant kernel timed with HIP events.  The allowed slowdown is loose on
purpose (boxes of one pool differ by several per cent and a record ages): the test is there to
catch a structural regression of a kernel or of the emitter, not drift.  The reference guards its
generated kernels the same way (``tests/perf/test_kernel_perf_regression.py:78-101``, threshold
1.25 against ``tests/perf/baselines/h100-80gb-hbm3.json``, skipped on any other GPU).

The nine registry operators are guarded too, as the reference guards exactly those kernels: each
operator's shipped single kernel at its tuned tiling, timed over a sample of its captured
workloads, the geometric mean against the record.

``CLEAVE_PERF_THRESHOLD`` overrides the allowed ratio.
"""

import json
import os

import pytest
import torch

from cleave_amd import examples as C
from cleave_amd.pipeline.direct import kernel_for

pytestmark = pytest.mark.gpu

THRESHOLD = float(os.environ.get("CLEAVE_PERF_THRESHOLD", "1.4"))
RECORD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "perf_mi355x.json")

ATTENTION = dict(HQ=32, HKV=8, SQ=4096, SKV=4096, D=64)
MATMUL = dict(M=4096, N=14336, K=4096)
# name -> (graded case whose program, element type and input builder are used, sizes, template, tiling, split)
PLANS = {
    "c1_matmul_128x128x4096": ("c1", C.FULL["c1"], "gemm_dma", dict(BM=16, BN=32, BK=64, WM=1, WN=1), 16),
    "c2_rmsnorm_matmul_16x11008x4096": ("c2", C.FULL["c2"], "skinny", dict(WAVES_N=1, WAVES_K=2), 8),
    "c3_gqa_decode_256h_8192": ("c3", C.FULL["c3"], "attn_decode", dict(WAVES=1, SKEW=30), 8),
    "c4_mla_decode_16x128h_4096": ("c4", C.FULL["c4"], "mla_decode", dict(DUO=1, LDS_AHEAD=4), 8),
    "matmul_4096x14336x4096": ("c1", MATMUL, "gemm_dma", dict(BM=256, BN=256, BK=64, WM=4, WN=2, TAIL=128), None),
    "attention_32h_4096_d64": ("c3", ATTENTION, "attn_prefill", dict(SHARED=1), None),
}
ROTATED_BYTES = 600 << 20          # input sets rotated per launch: well past the 256 MB last-level cache


@pytest.fixture(scope="module")
def record():
    with open(RECORD) as handle:
        stored = json.load(handle)
    found = torch.cuda.get_device_properties(0)
    device = f"{found.gcnArchName.split(':')[0]} with {found.multi_processor_count} compute units"
    if stored["device"] != device:
        pytest.skip(f"the record is for {stored['device']!r}, this GPU is {device!r}")
    return stored["operators"]


@pytest.mark.parametrize("name", sorted(PLANS))
def test_fixed_plan_latency(name, record):
    case, sizes, template, tiling, split = PLANS[name]
    program, dtype, make = C.CASES[case]
    traced = program.trace(dtype, **sizes)
    first = [t.cuda() for t in make(sizes, seed=70)]
    per_set = sum(t.numel() * t.element_size() for t in first)
    sets = [first] + [[t.cuda() for t in make(sizes, seed=71 + i)] for i in range(max(2, min(7, ROTATED_BYTES // per_set)))]
    kernel = kernel_for(traced, template=template, tiling=tiling, split=split)
    print(f"case perf guard {name}", flush=True)
    kernel(*sets[0])
    # (the matrix cores' clock settles over the first tenths of a second of load)
    heavy = record[name]["us"] > 100
    us = kernel.time(*sets[0], warmup=200 if heavy else 20, iters=100, rotate=sets[1:], only=[0]) * 1e3
    ratio = us / record[name]["us"]
    print(f"{name}: recorded {record[name]['us']:.1f} us, now {us:.1f} us ({ratio:.2f}x)", flush=True)
    assert ratio <= THRESHOLD, f"{name}: {us:.1f} us against the recorded {record[name]['us']:.1f} us ({ratio:.2f}x > {THRESHOLD}x)"


REGISTRY_WORKLOADS = 4        # workloads sampled per operator (first and last included)


def _registry_geomean(name):
    from cleave_amd.dynamic import OPERATORS
    from cleave_amd.runtime.autotune import geomean, time_kernel
    from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code

    op = OPERATORS[name]
    loaded = _load_main_kernel_from_code(op.kernel_source())
    kernel = _compile(loaded, loaded.manifest["out_idx"])
    times = {}
    for key, inputs, expected in op.keyed_workloads(keep=REGISTRY_WORKLOADS, dtype=torch.bfloat16)():
        got = kernel(*inputs)
        got = list(got) if isinstance(got, (list, tuple)) else [got]
        torch.cuda.synchronize()
        # (a guard of speed still refuses a kernel that has stopped being right)
        torch.testing.assert_close(got[0].float(), expected[0].float().to(got[0].device), rtol=2e-2, atol=2e-2)
        times[key] = time_kernel(kernel, inputs, warmup=10, iters=20, repeats=3)[0]
        del inputs, expected, got
        torch.cuda.empty_cache()
    return geomean(list(times.values())), times


def _registry_names():
    from cleave_amd.dynamic import OPERATORS

    return sorted(OPERATORS)


@pytest.mark.parametrize("name", _registry_names())
def test_registry_operator_latency(name, record):
    """Geometric mean over the sampled captured workloads of the operator's shipped kernel
    (``python/cleave/dynamic/registry.py:91-196`` names the same nine)."""
    print(f"case perf guard registry {name}", flush=True)
    now, times = _registry_geomean(name)
    want = record[name]["us"]
    ratio = now / want
    print(f"{name}: recorded geomean {want:.2f} us, now {now:.2f} us ({ratio:.2f}x); " +
          " ".join(f"{k}={v:.1f}" for k, v in times.items()), flush=True)
    assert ratio <= THRESHOLD, f"{name}: geomean {now:.2f} us against the recorded {want:.2f} us ({ratio:.2f}x > {THRESHOLD}x)"
