"""The C-ABI library loads and exports what the header declares; hiprtc compiles every template
without a GPU; host-side pipeline logic (specs, presets, saved kernels, ranking, grid
expressions); the validation evaluator agrees with the independent numpy oracle on CPU."""

import ctypes
import json
import re
from pathlib import Path

import numpy as np
import pytest
import torch

import cleave_amd
import cleave_amd.lang as cl
from cleave_amd.core.errors import CompileError, SpecError
from cleave_amd.runtime import shim
from cleave_amd import examples as C
from cleave_amd.pipeline.direct import source_for, stage_graph

ROOT = Path(__file__).resolve().parents[1]


def declared_symbols():
    text = (ROOT / "include" / "cleave_hip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"^\s*(?:const\s+)?[a-z_0-9]+\*?\s+\*?(chip_[a-z_]+)\s*\(", text, flags=re.M)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 14 and {"chip_compile", "chip_launch", "chip_launch_seq", "chip_time_launches",
                                 "chip_time_graph"} <= set(names)
    lib = shim.load()
    for n in names:
        assert hasattr(lib, n), f"libcleave_hip.so does not export {n}"
    assert lib.chip_abi_version() == shim.ABI_VERSION


def test_every_header_entry_cites_the_reference():
    text = (ROOT / "include" / "cleave_hip.h").read_text()
    for name in declared_symbols():
        head = text[:re.search(r"^[a-z][^\n]*\b" + name + r"\(", text, flags=re.M).start()]
        comment = head[head.rindex("\n/*"):]            # the last comment that starts a line
        assert re.search(r"python/cleave/[\w/]+\.py:\d+|no counterpart", comment), f"{name}: no reference citation"


def test_compile_error_carries_the_compiler_log():
    with pytest.raises(CompileError, match="undeclared_name"):
        shim.compile_source('extern "C" __global__ void k(int* p) { p[0] = undeclared_name; }', name="bad.hip")
    code, log = shim.compile_source('extern "C" __global__ void k(int* p) { p[0] = 1; }', name="ok.hip")
    assert code[:4] == b"\x7fELF"


@pytest.mark.parametrize("case,kw", [
    ("c1", dict(template="gemm", tiling=dict(BM=64, BN=64, BK=64, WM=2, WN=2), split=8)),
    ("c2", dict(template="skinny", tiling=dict(WAVES_N=1, WAVES_K=2), split=8)),
    ("c3", dict(template="attn_decode", tiling=dict(WAVES=2, PREFETCH=2), split=8)),
    ("c4", dict(template="mla_decode", tiling=dict(WAVES=4), split=8)),
])
def test_graded_configurations_compile_for_gfx950_without_a_gpu(case, kw):
    from cleave_amd.runtime.compile import compile_code_object

    fn, dt, _ = C.CASES[case]
    src = source_for(fn.trace(dt, **C.FULL[case]), **kw)
    assert "main_kernel_combine" in src
    assert compile_code_object(src)[:4] == b"\x7fELF"


def test_product_refuses_to_run_without_the_library(monkeypatch, tmp_path):
    from cleave_amd.core.errors import BackendUnavailable

    monkeypatch.setattr(shim, "_lib", None)
    monkeypatch.setenv("CLEAVE_HIP_LIBRARY", str(tmp_path / "libcleave_hip.so"))
    with pytest.raises(BackendUnavailable, match="libcleave_hip.so"):
        shim.load()
    with pytest.raises(BackendUnavailable):                      # and nothing else steps in for it
        shim.compile_source('extern "C" __global__ void k() {}', name="k.hip")


def test_grid_expressions_are_arithmetic_only():
    from cleave_amd.runtime.compile import eval_extent

    assert eval_extent("ceildiv(n_idx, 4) * batch + 1", dict(n_idx=10, batch=3)) == 10
    assert eval_extent(7, {}) == 7 and eval_extent("max(1, min(batch, 4))", dict(batch=9)) == 4
    for bad in ("__import__('os').system('true')", "batch.real", "(lambda: 1)()", "[1][0]", "open('x')"):
        with pytest.raises(CompileError):
            eval_extent(bad, dict(batch=1))
    with pytest.raises(CompileError, match="nope"):
        eval_extent("nope * 2", {})


# ----------------------------------------------------------------------------- specs
def test_paging_spec_refusals():
    from cleave_amd.dynamic.paging import (PAGED_DECODE, PAGED_DECODE_SLAB, CombineTiling, InvalidSpec, MLASpec,
                                           PagingSpec)

    PagingSpec(32, 8).validate()
    PagingSpec(32, 8, kind=PAGED_DECODE_SLAB, page_size=64).validate()
    for bad, msg in [(PagingSpec(32, 5), "do not divide"), (PagingSpec(8, 1), "single kv head"),
                     (PagingSpec(8, 8), "group"), (PagingSpec(32, 8, page_size=64), "slab access layer"),
                     (PagingSpec(32, 8, kind=PAGED_DECODE_SLAB), "degenerate"),
                     (PagingSpec(32, 8, kind="nonesuch"), "unknown access layer|slab"),
                     (PagingSpec(32, 8, causal=True), "causal"),
                     (PagingSpec(32, 8, query_input="K_CACHE"), "collide"),
                     (PagingSpec(32, 8, grid_order=("head", "head")), "grid_order"),
                     (PagingSpec(32.0, 8), "must be an int")]:
        with pytest.raises(InvalidSpec, match=msg):
            bad.validate()
    CombineTiling(8, split_step=2, cols=64).validate(128)
    for bad in (CombineTiling(1), CombineTiling(8, split_step=3), CombineTiling(8, cols=48), CombineTiling(8, loop_kind="x")):
        with pytest.raises(InvalidSpec):
            bad.validate(128)
    MLASpec(128).validate() if hasattr(MLASpec(128), "validate") else None


def test_only_the_registered_paged_layers_are_built():
    from cleave_amd.dynamic import registry
    from cleave_amd.dynamic.paging import (RAGGED_PREFILL_CAUSAL, DenseAttention, PagingSpec, UnsupportedTiling,
                                           apply_paging_split, build_split_decode, CombineTiling)

    assert "gqa_paged_decode_h32_kv8_d128_ps64" in registry.OPERATORS
    spec = PagingSpec(32, 32 // 4, kind=RAGGED_PREFILL_CAUSAL, causal=True)
    with pytest.raises(UnsupportedTiling):
        build_split_decode(spec, DenseAttention(16, 32, 128, 256, "float16", "float16", waves=4), 8, CombineTiling(8))


def test_paged_mla_layer_plans_and_signature():
    """The paged MLA decode layer: the single kernel and the chunked split pair carry the
    reference operator's argument order, the item count and item size are launch-time
    expressions over the table length, and what is not built is refused by name."""
    from cleave_amd.codegen import HipCodeGen, parse_manifest
    from cleave_amd.dynamic import registry
    from cleave_amd.dynamic.paging import (MLA_PAGED_PREFILL_CAUSAL, CombineTiling, DenseAttention, DenseMLA, MLASpec,
                                           NotDenseAttention, UnsupportedTiling, build_split_decode)

    op = registry.OPERATORS["mla_paged_decode_h16_ckv512_kpe64_ps1"]
    assert op.is_mla and op.scale == pytest.approx(0.1352337747812271) and len(op.workloads) == 4
    m = parse_manifest(op.kernel_source())
    assert [p["name"] for p in m["params"]] == ["PlaceHolder_QN", "PlaceHolder_QP", "PlaceHolder_CKV", "PlaceHolder_KPE",
                                               "PlaceHolder_KV_INDPTR", "PlaceHolder_KVI", "sm_scale", "OutputNode_0",
                                               "OutputNode_1"]
    by = {p["name"]: p for p in m["params"]}
    assert by["PlaceHolder_CKV"]["shape"] == ["num_pages", 1, 512] and by["OutputNode_1"]["dtype"] == "float32"
    assert m["launches"][0]["grid"] == ["batch", "1", "1"] and m["launches"][0]["block"][0] == 64
    spec, dense = MLASpec(num_qo_heads=32), DenseMLA(32, 512, 64, "bfloat16", "bfloat16")
    pair = parse_manifest(HipCodeGen().gen(build_split_decode(spec, dense, 8, CombineTiling(split=8))))
    assert [l["entry"] for l in pair["launches"]] == ["main_kernel", "main_kernel_combine"]
    assert pair["launches"][0]["grid"][:2] == ["ceildiv(n_idx, chunk_pages) + batch", "2"]
    assert dict(pair["derived_dims"])["chunk_pages"].startswith("max(32, min(512, ceildiv(n_idx")
    scratch = {p["name"]: p for p in pair["params"] if p["role"] == "scratch"}
    assert scratch["Partial_PO_split"]["shape"] == ["ceildiv(n_idx, chunk_pages) + batch", 32, 512]
    with pytest.raises(UnsupportedTiling, match="decode transformation"):
        build_split_decode(MLASpec(16, kind=MLA_PAGED_PREFILL_CAUSAL, causal=True), DenseMLA(16, 512, 64, "bfloat16", "bfloat16"),
                           8, CombineTiling(split=8))
    pre = parse_manifest(registry.OPERATORS["mla_paged_prefill_causal_h16_ckv512_kpe64_ps1"].kernel_source())
    assert [p["name"] for p in pre["params"]] == ["PlaceHolder_Q_NOPE", "PlaceHolder_Q_PE", "PlaceHolder_CKV_CACHE",
                                                 "PlaceHolder_KPE_CACHE", "PlaceHolder_QO_INDPTR", "PlaceHolder_KV_INDPTR",
                                                 "PlaceHolder_KV_INDICES", "sm_scale", "OutputNode_0", "OutputNode_1"]
    # two query tokens (waves) per work item: a new item at every second packed token and at every request boundary
    assert pre["launches"][0]["grid"][0] == "ceildiv(total_q, 2) + batch" and pre["launches"][0]["block"][0] == 128
    assert dict(pre["derived_dims"]) == {"batch": "len_indptr - 1"} and pre["tiling"]["TOK"] == 2
    gqa = parse_manifest(registry.OPERATORS["gqa_ragged_prefill_causal_h32_kv8_d128"].kernel_source())
    assert [p["name"] for p in gqa["params"]] == ["PlaceHolder_Q", "PlaceHolder_K", "PlaceHolder_V", "PlaceHolder_QO_INDPTR",
                                                 "PlaceHolder_KV_INDPTR", "sm_scale", "OutputNode_0", "OutputNode_1"]
    # the operator's own kernel is the one whose four waves share key tiles through LDS (128 rows = 32 tokens x 4)
    # (the item axis is padded to a multiple of 8: one contiguous eighth of the space per XCD)
    assert gqa["launches"][0]["grid"][:2] == ["ceildiv(ceildiv(total_q, 32) + batch, 8) * 8", "8"]
    assert gqa["launches"][0]["block"][0] == 256
    from cleave_amd.dynamic.paging import RAGGED_PREFILL_CAUSAL, PagingSpec
    from cleave_amd.dynamic.paging.apply import _prefill_plan

    spec = PagingSpec(32, 8, kind=RAGGED_PREFILL_CAUSAL, causal=True, cache_inputs=("K", "V"))
    rows16 = parse_manifest(HipCodeGen().gen(_prefill_plan(spec, DenseAttention(16, 32, 128, 512, "bfloat16", "bfloat16",
                                                                                waves=8), shared=False)))
    assert rows16["launches"][0]["grid"][0] == "ceildiv(total_q, 4) + batch" and rows16["launches"][0]["block"][0] == 512
    assert set(registry.OPERATORS) >= {"gqa_paged_prefill_causal_h32_kv8_d128_ps1", "gqa_paged_prefill_causal_h32_kv4_d128_ps1",
                                       "gqa_ragged_prefill_causal_h32_kv4_d128"} and len(registry.OPERATORS) == 9
    with pytest.raises(NotDenseAttention, match="same operator family"):
        build_split_decode(MLASpec(16), DenseAttention(16, 32, 128, 256, "bfloat16", "bfloat16"), 8, CombineTiling(split=8))
    with pytest.raises(UnsupportedTiling, match="heads"):
        build_split_decode(MLASpec(32), DenseMLA(16, 512, 64, "bfloat16", "bfloat16"), 8, CombineTiling(split=8))


def test_presets_and_configs():
    from cleave_amd.pipeline.config import (EvalConfig, ScheduleConfig, SuperoptConfig, auto_max_ops, get_preset,
                                            list_presets)

    assert set(list_presets()) == {"fast", "default", "exhaustive"}
    assert get_preset("default").schedule.topk == 1000 and get_preset("default").eval.iters == 1000
    assert get_preset("fast").eval.replace(iters=7).iters == 7
    assert auto_max_ops(3, 1, False) == 13 and auto_max_ops(14, 1, True) == 18
    assert SuperoptConfig(split="K").split == ("K",) and ScheduleConfig(split_k=[4, 8]).split_k == (4, 8)
    prog = C.gqa_decode_exact.trace(cl.f16, **C.FULL["c3"])
    assert SuperoptConfig(split=("SKV",)).resolve_max_ops(prog) == auto_max_ops(prog.op_count, 1, True)
    for bad in (lambda: get_preset("warp"), lambda: ScheduleConfig(fusion="maybe"), lambda: ScheduleConfig(topk=0),
                lambda: SuperoptConfig(max_ops=0)):
        with pytest.raises(SpecError):
            bad()


def test_saved_kernel_round_trip(tmp_path):
    from cleave_amd.pipeline.kernel import Kernel, Param, Stage, load

    prog = C.matmul.trace(cl.f16, **C.FULL["c1"])
    fused = source_for(prog, template="gemm", tiling=dict(BM=64, BN=64, BK=64, WM=2, WN=2))
    st = Stage("main", fused, [-1], [Param("PlaceHolder_x", "input", 0, (128, 4096)),
                                     Param("PlaceHolder_w", "input", 1, (4096, 128))], "gemm 64x64", 6.5)
    k = Kernel([st], name="matmul", input_names=["x", "w"], input_shapes=[(128, 4096), (4096, 128)],
               output_shapes=[(128, 128)], variant="solo", label="gemm 64x64", latency_us=6.5)
    d = k.save(tmp_path / "k")
    meta = json.loads((d / "kernel.json").read_text())
    assert meta["format"] == 1 and meta["stages"][0]["file"] == "kernel.hip" and (d / "kernel.hip").read_text() == fused
    back = load(d)
    assert (back.name, back.variant, back.latency_us, back.input_names) == ("matmul", "solo", 6.5, ["x", "w"])
    assert back.stages[0].params == st.params and back.source == fused and back.meta["loaded_from"] == str(d)
    with pytest.raises(TypeError, match="expected 2 inputs"):
        back(torch.zeros(128, 4096))
    with pytest.raises(ValueError, match="shape"):
        back(torch.zeros(128, 4095), torch.zeros(4096, 128))
    meta["format"] = 9
    (d / "kernel.json").write_text(json.dumps(meta))
    with pytest.raises(ValueError, match="unsupported kernel format"):
        load(d)


def test_ranking_picks_the_fastest_eligible_candidate():
    from cleave_amd.runtime.autotune import WorkloadCandidate, format_ranking, geomean, pick_best, rank, sampled

    a = WorkloadCandidate("a", "", latency_us={"w1": 10.0, "w2": 40.0})
    b = WorkloadCandidate("b", "", latency_us={"w1": 30.0, "w2": 30.0})
    ref = WorkloadCandidate("tuned", "", origin="tuned (reference)", tuned=True, eligible=False,
                            latency_us={"w1": 5.0, "w2": 5.0})
    assert geomean([10.0, 40.0]) == pytest.approx(20.0) and a.geomean_us == pytest.approx(20.0)
    ranked = rank([b, a, ref])
    assert [c.label for _, c in ranked] == ["tuned", "a", "b"] and pick_best(ranked) is a
    text = format_ranking([a, b, ref])
    assert "winner: a" in text and "does NOT dominate" in text
    with pytest.raises(ValueError, match="No eligible"):
        pick_best(rank([ref]))
    with pytest.raises(ValueError, match="No correct"):
        pick_best([])
    assert WorkloadCandidate("x", "").geomean_us == float("inf")
    assert len(list(sampled(list(range(100)), 10))) == 10 and list(sampled([1, 2], 0)) == [1, 2]


def test_selected_candidates_are_held_to_the_strict_bound():
    from cleave_amd.pipeline.config import EvalConfig
    from cleave_amd.pipeline.build import resolve_tolerance
    from cleave_amd.runtime.validate import STRICT_TOLERANCE, Tolerance

    assert (STRICT_TOLERANCE.rtol, STRICT_TOLERANCE.atol) == (1e-2, 1e-2)
    assert resolve_tolerance(EvalConfig()) == STRICT_TOLERANCE            # the pipeline default, not the loose bound
    assert resolve_tolerance(EvalConfig(tolerance=Tolerance(1e-3, 1e-3))).rtol == 1e-3


# ----------------------------------------------------------------------------- evaluator vs oracle (CPU)
@pytest.mark.parametrize("case", ["c1", "c2", "c3", "c4"])
def test_validation_evaluator_agrees_with_the_numpy_oracle(case):
    """Two independent restatements (torch evaluator used to validate candidates; numpy oracle
    used by the tests) of the same program must agree on small shapes."""
    from cleave_amd.runtime.reference import execute
    from oracle import program_oracle

    fn, dt, make_inputs = C.CASES[case]
    prog = fn.trace(dt, **C.SMALL[case])
    inputs = make_inputs(C.SMALL[case], seed=5)
    want = program_oracle.evaluate(prog, inputs)[0]
    got = execute(stage_graph(prog), inputs)[0].float().numpy().reshape(want.shape)
    np.testing.assert_allclose(got, want, rtol=1e-2, atol=1e-2)


def test_saved_paged_kernel_holds_its_program_as_json(tmp_path):
    """A paged operator's directory is plain data: program.json + sources + dispatch.json.  It
    loads back to the same operator, and a directory that names a pickle is refused unread."""
    import json

    import cleave_amd.lang as cl
    from cleave_amd import examples
    from cleave_amd.frontend.paged import trace_paged
    from cleave_amd.pipeline import load
    from cleave_amd.pipeline.dynamic import PagedKernel

    attention = trace_paged(examples.paged_decode_op(32, 8, 128, 64, dtype=cl.bf16, name="op")).attention()
    kernel = PagedKernel(attention, attention.paging_spec(), "// main", label="L", variant="solo", latency_us=1.5,
                         dispatch={"min_tiles": 3, "geomean_us": {"hybrid": 1.0}},
                         dispatch_sources={"split": "// pair", "single": "// one"})
    folder = kernel.save(tmp_path / "k")
    assert {"program.json", "kernel.json", "kernel.hip", "dispatch.json", "dispatch.split.hip"} <= {p.name for p in folder.iterdir()}
    assert not list(folder.glob("*.pkl"))
    back = load(folder)
    assert isinstance(back, PagedKernel) and back.spec == kernel.spec and back.source == "// main"
    assert back.dispatch["min_tiles"] == 3 and back.dispatch_sources == kernel.dispatch_sources
    assert [p.name for p in back.attention.inputs] == [p.name for p in attention.inputs]
    # the host-side dispatch rule: kv tiles of the longest request against the calibrated threshold
    back.dispatch.update(page_size=64, kv_tile=32)
    assert back.dispatch_role(1) == "single" and back.dispatch_role(2) == "split"       # 64 tokens = 2 tiles < 3 <= 4 tiles
    document = json.loads((folder / "kernel.json").read_text())
    document["paged"] = "program.pkl"
    (folder / "kernel.json").write_text(json.dumps(document))
    (folder / "program.pkl").write_bytes(b"not read")
    with pytest.raises(ValueError, match="pickle"):
        load(folder)


def test_partials_of_a_kernel_that_cuts_the_keys_its_own_way_are_compared_through_their_fold():
    """Softmax partials (m, l, O) of any partition of the keys fold to the same (lse, O / l); per split they
    differ.  A kernel whose manifest says it skews its ranges is validated through the fold."""
    from cleave_amd.runtime.validate import _comparable, own_cut

    gen = torch.Generator().manual_seed(3)
    s, v = torch.randn(6, 4, 512, generator=gen) * 3, torch.randn(6, 512, 64, generator=gen)

    def parts(cuts):
        pm, pl, po = [], [], []
        for lo, hi in cuts:
            if hi <= lo:
                pm.append(torch.full((6, 4), -1.0e30)); pl.append(torch.zeros(6, 4)); po.append(torch.zeros(6, 4, 64))
                continue
            blk = s[..., lo:hi]
            m = blk.amax(-1)
            w = torch.exp2(blk - m.unsqueeze(-1))
            pm.append(m + 3.0); pl.append(w.sum(-1) / 8.0); po.append(w @ v[:, lo:hi] / 8.0)   # (any reference point)
        n = len(cuts)
        return [torch.stack(pm).reshape(n, 24), torch.stack(pl).reshape(n, 24), torch.stack(po).reshape(n, 24, 64)]

    equal = parts([(0, 128), (128, 256), (256, 384), (384, 512)])
    skewed = parts([(0, 160), (160, 256), (256, 512), (512, 512)])
    for a, b in zip(_comparable(equal, "softmax_partial_folded"), _comparable(skewed, "softmax_partial_folded")):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)
    per_split = [float((a - b).abs().max()) for a, b in zip(_comparable(equal, "softmax_partial"), _comparable(skewed, "softmax_partial"))]
    assert max(per_split) > 0.1
    whole = torch.softmax(s * 0.6931471805599453, -1) @ v
    torch.testing.assert_close(_comparable(skewed, "softmax_partial_folded")[1], whole.reshape(24, 64), rtol=1e-4, atol=1e-4)

    class K:
        manifest = {"tiling": {"WAVES": 1, "SKEW": 30}}

    assert own_cut(K) and not own_cut(type("P", (), {"manifest": {"tiling": {"WAVES": 1}}}))


def test_token_threshold_of_the_prefill_dispatch():
    """The rule "the other kernel up to T query tokens" is chosen by the geometric mean over the
    workloads: a threshold only where the other kernel wins on every workload below it by enough
    to pay for those it loses, and none when the winner is better everywhere."""
    from cleave_amd.pipeline.dynamic import pick_token_threshold

    tokens = {"a": 1, "b": 34, "c": 969, "d": 16294}
    winner = {"a": 4.0, "b": 5.5, "c": 10.0, "d": 170.0}
    small = {"a": 3.4, "b": 5.0, "c": 14.0, "d": 600.0}
    t, us = pick_token_threshold(winner, small, tokens)
    assert t == 34 and us < (4.0 * 5.5 * 10.0 * 170.0) ** 0.25
    mixed = {"a": 6.0, "b": 5.0, "c": 14.0, "d": 600.0}          # loses on the smallest, wins on the next
    t, us = pick_token_threshold(winner, mixed, tokens)
    assert t is None and abs(us - (4.0 * 5.5 * 10.0 * 170.0) ** 0.25) < 1e-9
    t, _ = pick_token_threshold(winner, {"a": 3.0, "b": 9.0, "c": 14.0, "d": 600.0}, tokens)
    assert t == 1
    assert pick_token_threshold(winner, {"x": 1.0}, tokens) == (None, float("inf"))
