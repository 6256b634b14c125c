"""The stored superoptimizer structures the reference calls valid
(``tests/integration/graph_structures/*/before_split_*valid*.graph`` and the split-K matmul), with
their symbolic extents mapped to real sizes, lowered, tiled by the search, generated, compiled and
run; the expected values come from running the stored ops one at a time in float64 on the same
f16 inputs.  A structure that carries split ops is built as partial + combine at its own split
count, wherever in the graph the superoptimizer put the split."""

import json

import numpy as np
import pytest
import torch

from cleave_amd.codegen import HipCodeGen
from cleave_amd.ir import to_ir as flat_ir
from cleave_amd.lower import to_ir
from cleave_amd.lower.stages import split_stages
from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code
from cleave_amd.schedule import apply_tiling, search_tiling
from tests.test_stored_structures import STRUCT, VALID, interpret

pytestmark = pytest.mark.gpu

SIZES = {"gqa": {8: 16, 4: 8, 16: 512, 20: 64},            # 16 query heads over 8 kv heads, 12 rows, 512 keys, d = 64
         "rmsnorm": {4: 16, 8: 512, 12: 4096},
         "matmul": {4: 64, 8: 256, 12: 1024}}


@pytest.mark.parametrize("name", VALID)
def test_valid_stored_structure_runs_against_its_own_ops(name):
    sizes = SIZES["gqa" if "_gqa_" in name else "rmsnorm" if "rmsnorm" in name else "matmul"]
    structure = json.loads((STRUCT / name).read_text())
    graph = to_ir(structure, symbol_map=sizes, dtype="float16")
    splits = {n.shape[0] for n in graph.nodes if getattr(n, "op", None) == "split"}
    print(f"case {name}: {graph.lowered.family} {graph.lowered.problem} splits {splits}", flush=True)
    if splits:
        part, comb = split_stages(graph, splits.pop())
        source = HipCodeGen().gen([apply_tiling(search_tiling(part)[0]), apply_tiling(search_tiling(comb)[0])])
    else:
        source = HipCodeGen().gen(apply_tiling(search_tiling(graph)[0]))
    loaded = _load_main_kernel_from_code(source)
    kernel = _compile(loaded, loaded.manifest["out_idx"])
    gen = torch.Generator().manual_seed(7)
    inputs = [(torch.randn(p.shape, generator=gen) * (0.05 if "rmsnorm" in name or "matmul" in name else 1.0)).half()
              for p in graph.placeholders]
    got = kernel(*[t.cuda() for t in inputs])
    got = (got[0] if isinstance(got, (tuple, list)) else got).float().cpu().numpy()
    flat = flat_ir(structure, symbol_map=sizes, dtype="float16")
    want, = interpret(flat, {p.name: t.double().numpy() for p, t in zip(flat.placeholders, inputs)}, check_shapes=False)
    np.testing.assert_allclose(got.reshape(want.shape), want, rtol=1e-2, atol=1e-2)
