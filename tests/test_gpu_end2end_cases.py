"""The reference's end-to-end case list, name by name at its sizes
(``tests/schedule/end2end/test_end2end.py:14-43``; the table is ``tests/_end2end_cases.py``): every
case is traced, lowered, searched (``search_tiling``) and its best candidates are compiled, checked
against the torch evaluation of the graph at rtol = atol = 1e-2 and timed by ``run_candidates``
in child processes -- the reference's ``run_end2end_candidates``
(``tests/schedule/end2end/_test_utils.py:13-60``).

The tiling space is this back end's own, so the reference's success counts do not carry over: a
case passes when candidates exist, every one of the best ``TOPK`` validates, and none fails for
a reason other than a tiling the emitter refuses.
"""

import pytest
import torch

from cleave_amd.runtime import workers
from cleave_amd.runtime.evaluate import run_candidates
from cleave_amd.runtime.validate import BenchOptions
from cleave_amd.schedule import search_tiling

from ._end2end_cases import CASES, flat_graph

pytestmark = pytest.mark.gpu

TOPK = 8


@pytest.fixture(scope="module")
def pool():
    with workers.WorkerPool() as shared:
        yield shared


@pytest.mark.parametrize("name", sorted(CASES))
def test_end2end(name, pool):
    candidates = search_tiling(flat_graph(name), topk=TOPK)
    assert candidates, "the search proposes nothing for this case"
    print(f"case {name}: {len(candidates)} candidates", flush=True)
    results = run_candidates(candidates, "float16", max_parallel=4, pool=pool, benchmark=BenchOptions(2, 5))
    torch.cuda.synchronize()
    refused = [r for r in results if not r.ok and r.stage == "codegen"]
    wrong = [r for r in results if not r.ok and r.stage != "codegen"]
    assert not wrong, "\n".join(f"{r.label}: {r.stage}: {r.error}" for r in wrong)
    assert len(results) > len(refused), "every candidate was refused by the emitter"
    assert all(r.latency_ms and r.latency_ms > 0 for r in results if r.ok)
    print(f"case {name}: {len(results) - len(refused)} validated, {len(refused)} refused by the emitter, "
          f"best {min(r.latency_ms for r in results if r.ok) * 1e3:.1f} us", flush=True)
