"""The stored superoptimizer structures the reference calls valid
(``tests/integration/graph_structures/*/before_split_*valid*.graph`` and the split-K matmul), with
their symbolic extents mapped to real sizes, lowered, tiled by the search, generated, compiled and
run; the expected values come from running the stored ops one at a time in float64 on the same
f16 inputs.  A structure that carries split ops is built as partial + combine at its own split
count, wherever in the graph the superoptimizer put the split; the [partial, combine] pairs the
reference's split pass makes of them (``after_split_*``) go the same way."""

import json

import numpy as np
import pytest
import torch

from cleave_amd.codegen import HipCodeGen
from cleave_amd.ir import to_ir as flat_ir
from cleave_amd.lower import to_bundles
from cleave_amd.lower.stages import join_cut_pair
from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code
from cleave_amd.schedule import apply_tiling, search_tiling
from tests.test_stored_structures import AFTER, STRUCT, VALID, interpret

pytestmark = pytest.mark.gpu

SIZES = {"gqa": {8: 16, 4: 8, 16: 512, 20: 64},            # 16 query heads over 8 kv heads, 12 rows, 512 keys, d = 64
         "rmsnorm": {4: 16, 8: 512, 12: 4096},
         "matmul": {4: 64, 8: 256, 12: 1024}}


@pytest.mark.parametrize("name", VALID + [n for n in AFTER if "invalid" not in n])
def test_valid_stored_structure_runs_against_its_own_ops(name):
    sizes = SIZES["gqa" if "_gqa_" in name else "rmsnorm" if "rmsnorm" in name else "matmul"]
    structure = json.loads((STRUCT / name).read_text())
    flat = flat_ir(join_cut_pair(*structure) if isinstance(structure[0], list) else structure, symbol_map=sizes, dtype="float16")
    splits = {n.shape[0] for n in flat.ops if n.op == "split"}
    stages, = to_bundles([structure], symbol_map=sizes, split_factors=sorted(splits) or None, dtype="float16")
    graph = stages[0]
    print(f"case {name}: {graph.lowered.family} {graph.lowered.problem} splits {splits}", flush=True)
    assert len(stages) == (2 if splits else 1)
    source = HipCodeGen().gen([apply_tiling(search_tiling(g)[0]) for g in stages] if splits else apply_tiling(search_tiling(graph)[0]))
    loaded = _load_main_kernel_from_code(source)
    kernel = _compile(loaded, loaded.manifest["out_idx"])
    gen = torch.Generator().manual_seed(7)
    inputs = [(torch.randn(p.shape, generator=gen) * (0.05 if "rmsnorm" in name or "matmul" in name else 1.0)).half()
              for p in flat.placeholders]
    got = kernel(*[t.cuda() for t in inputs])
    got = (got[0] if isinstance(got, (tuple, list)) else got).float().cpu().numpy()
    want, = interpret(flat, {p.name: t.double().numpy() for p, t in zip(flat.placeholders, inputs)}, check_shapes=False)
    np.testing.assert_allclose(got.reshape(want.shape), want, rtol=1e-2, atol=1e-2)
