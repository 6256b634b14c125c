"""Lowering of op-dict structures (the reference's stored superoptimizer output as data),
operator recognition, the gfx950 schedule space, and what the emitter writes."""

import json
from pathlib import Path

import pytest

import cleave_amd.lang as cl
from cleave_amd.codegen import HipCodeGen, parse_manifest
from cleave_amd.core.errors import CodegenError, LoweringRejected, ScheduleRejected
from cleave_amd.ir import recognize, to_ir
from cleave_amd.lower import to_bundles
from cleave_amd.lower.stages import partial_buffers, split_stages
from cleave_amd.schedule import apply_tiling, search_tiling
from cleave_amd.schedule.hint import TileDict
from cleave_amd import examples as C
from cleave_amd.pipeline.direct import source_for, stage_graph

STRUCT = Path(__file__).parent / "golden" / "graph_structures"


def stored(name, **kw):
    return to_ir(json.loads((STRUCT / name).read_text()), dtype="float16", **kw)


def test_stored_split_k_matmul_is_read_through_its_split_ops():
    low = recognize(stored("before_split_matmul_split_k_graph_structure.graph"))
    assert low.family == "matmul" and low.split_dim == "K"
    assert (low.problem["M"], low.problem["N"], low.problem["K"]) == (4, 8, 12)
    assert sorted(low.split_axes.values()) == [0, 1]            # A split on its K axis (1), B on its K axis (0)


def test_stored_reordered_rmsnorm_matmul_is_recognised():
    """The superoptimizer's (x @ w) * rsqrt(sum(x*x)/K) form, symbolic extents mapped to real ones."""
    low = recognize(stored("before_split_rmsnorm_matmul_graph_structure_valid_1.graph", symbol_map={12: 4096}))
    assert low.family == "rmsnorm_matmul" and low.problem["K"] == 4096 and low.problem["eps"] == 0.0
    assert not low.problem["gamma"] and set(low.operands) == {"A", "B"}


def test_stored_split_gqa_is_attention_split_over_kv():
    low = recognize(stored("before_split_gqa_graph_structure_valid_1.graph"))
    p = low.problem
    assert low.family == "attention" and low.split_dim == "SKV"
    assert (p["units"], p["group"], p["sq"], p["skv"], p["head_dim"]) == (4, 2, 12, 16, 20)
    assert p["scale"] == pytest.approx(1 / 8.0) and p["shift"] == -6.25 and not p["exact"]


@pytest.mark.parametrize("name", ["before_split_rmsnorm_matmul_graph_structure_invalid_1.graph",
                                  "before_split_rmsnorm_matmul_graph_structure_invalid_3.graph",
                                  "before_split_gqa_graph_structure_invalid_2.graph",
                                  "before_split_gqa_graph_structure_invalid_3.graph"])
def test_stored_invalid_splits_are_refused(name):
    with pytest.raises(LoweringRejected):
        recognize(stored(name, symbol_map={12: 4096}))


def test_cut_pair_structure_parses_but_is_not_a_single_operator():
    pair = json.loads((STRUCT / "after_split_matmul_split_k_graph_structure.graph").read_text())
    partial, combine = (to_ir(s, dtype="float16") for s in pair)
    assert partial.op_kinds() == ["split", "split", "matmul"] and combine.op_kinds() == ["reduce_sum"]
    with pytest.raises(LoweringRejected):
        recognize(partial)      # its output still carries the split axis: a cut partial is not a whole operator


@pytest.mark.parametrize("case,family", [("c1", "matmul"), ("c2", "rmsnorm_matmul"), ("c3", "attention"), ("c4", "mla")])
def test_graded_programs_map_to_their_families(case, family):
    fn, dt, _ = C.CASES[case]
    g = stage_graph(fn.trace(dt, **C.FULL[case]))
    assert g.lowered.family == family
    if case == "c2":
        assert g.lowered.problem["gamma"] and g.lowered.problem["eps"] == pytest.approx(1e-6)
    if case == "c3":
        assert g.lowered.problem["exact"] and (g.lowered.problem["units"], g.lowered.problem["group"]) == (64, 4)
    if case == "c4":
        assert g.lowered.problem["scale"] == pytest.approx(192 ** -0.5)


def test_swiglu_is_a_family_of_its_own():
    """``(x @ w_up) * silu(x @ w_gate)`` in either operand order: A the shared activation, B the
    bare product's weight, C the weight under the silu; tilings of the direct-to-LDS matmul whose
    B tile holds the same columns of both weights; no split-K form."""
    import cleave_amd

    shapes = dict(M=4096, N=14336, K=4096)
    g = stage_graph(C.swiglu.trace(cl.f16, **shapes))
    low = g.lowered
    assert low.family == "swiglu" and (low.problem["M"], low.problem["N"], low.problem["K"]) == (4096, 14336, 4096)
    assert {r: n.name for r, n in low.operands.items()} == {"A": "PlaceHolder_x", "B": "PlaceHolder_w_up",
                                                            "C": "PlaceHolder_w_gate"}

    @cleave_amd.jit
    def flipped(x: cl.Tensor["M", "K"], w_gate: cl.Tensor["K", "N"], w_up: cl.Tensor["K", "N"]):
        return cl.silu(x @ w_gate) * (x @ w_up)

    low2 = stage_graph(flipped.trace(cl.f16, **shapes)).lowered
    assert low2.family == "swiglu" and low2.operands["C"].name == "PlaceHolder_w_gate"

    cands = search_tiling(g, topk=10_000)
    assert cands and {c.template for c in cands} == {"gemm_dma"}
    for c in cands:
        t = c.tiling
        assert t["SWIGLU"] == 1 and (t["BN"] // t["WN"] // 16) % 2 == 0 and c.output_tile == [t["BM"], t["BN"] // 2]
    m = parse_manifest(source_for(C.swiglu.trace(cl.f16, **shapes), template="gemm_dma",
                                  tiling=dict(BM=256, BN=256, BK=64, WM=4, WN=2, SWIGLU=1)))
    assert [p["name"] for p in m["params"]] == ["PlaceHolder_x", "PlaceHolder_w_up", "PlaceHolder_w_gate", "OutputNode_0"]
    assert m["launches"][0]["grid"] == ["112", "16", "1"]          # 14336 / (256 / 2) column tiles
    with pytest.raises(LoweringRejected, match="no split form"):
        split_stages(g, 4)


def test_matmul_rowsum_is_a_family_of_its_own():
    g = stage_graph(C.matmul_rowsum.trace(cl.f16, **C.FULL["matmul_rowsum"]))
    assert g.lowered.family == "matmul_rowsum" and g.outputs[0].shape == (4096, 1)
    cands = search_tiling(g, topk=10_000)
    assert cands and all(c.template == "gemm_dma" and c.tiling["ROWSUM"] == 1 and 4096 % c.tiling["BN"] == 0 for c in cands)
    m = parse_manifest(source_for(C.matmul_rowsum.trace(cl.f16, **C.FULL["matmul_rowsum"]), template="gemm_dma",
                                  tiling=dict(BM=16, BN=256, BK=64, WM=1, WN=4, ROWSUM=1)))
    assert m["launches"][0]["grid"] == ["1", "256", "1"]           # one workgroup per 16 rows walks all of N
    with pytest.raises(LoweringRejected, match="no split form"):
        split_stages(g, 2)


def test_qk_norm_attention_is_attention_with_normalised_operands():
    g = stage_graph(C.qknorm.trace(cl.f16, HQ=64, HKV=8, SQ=4096, SKV=4096, D=128))
    low = g.lowered
    assert low.family == "attention" and low.problem["norm_eps"] == {"q": pytest.approx(1e-6), "k": pytest.approx(1e-6)}
    assert (low.problem["units"], low.problem["group"]) == (8, 8)
    assert {c.template for c in search_tiling(g, topk=100)} == {"attn_prefill"}     # the streaming kernel has no norm form
    with pytest.raises(ScheduleRejected, match="many-row kernel"):
        search_tiling(stage_graph(C.qknorm.trace(cl.f16, HQ=4, HKV=4, SQ=1, SKV=256, D=384)))
    # the first candidate normalises the keys once, by a launch of its own into a scratch copy the attention kernel reads
    m = parse_manifest(source_for(C.qknorm.trace(cl.f16, HQ=64, HKV=8, SQ=4096, SKV=4096, D=128)))
    assert [launch["entry"] for launch in m["launches"]] == ["main_kernel_keys", "main_kernel"]
    assert m["launches"][0]["args"] == ["PlaceHolder_k", "Scratch_kn"] and m["launches"][0]["grid"] == ["2048", "1", "1"]
    assert m["launches"][1]["args"] == ["PlaceHolder_q", "PlaceHolder_k", "PlaceHolder_v", "Scratch_kn", "OutputNode_0"]
    assert [p["role"] for p in m["params"]] == ["input", "input", "input", "scratch", "output"]
    m = parse_manifest(source_for(C.qknorm.trace(cl.f16, HQ=64, HKV=8, SQ=4096, SKV=4096, D=128), template="attn_prefill",
                                  tiling=dict(SHARED=1)))
    assert m["launches"][0]["grid"] == ["256", "8", "1"] and m["launches"][0]["block"][0] == 256


def test_lora_is_a_family_of_its_own():
    g = stage_graph(C.lora.trace(cl.f16, **C.FULL["lora"]))
    low = g.lowered
    assert low.family == "lora" and low.problem["R"] == 16
    assert {r: n.name for r, n in low.operands.items()} == {"A": "PlaceHolder_x", "B": "PlaceHolder_w",
                                                            "LA": "PlaceHolder_a", "LB": "PlaceHolder_b"}
    cands = search_tiling(g, topk=100)
    assert cands and all(c.template == "skinny" and c.tiling["LORA"] == 1 for c in cands)
    m = parse_manifest(source_for(C.lora.trace(cl.f16, **C.FULL["lora"])))
    assert [p["name"] for p in m["params"]] == ["PlaceHolder_x", "PlaceHolder_w", "PlaceHolder_a", "PlaceHolder_b",
                                                 "OutputNode_0"]
    with pytest.raises(ScheduleRejected, match="few-row matmul kernel only"):
        search_tiling(stage_graph(C.lora.trace(cl.f16, M=256, N=512, K=512, R=16)))
    # split over K: partial sums of both products; the combine applies the rank update, so it also reads the up factor
    partial, combine = split_stages(g, 8)
    assert [o.shape for o in partial.outputs] == [(8, 16, 4096), (8, 16, 16)]
    assert [p.name for p in combine.placeholders] == ["PlaceHolder_PACC", "PlaceHolder_PD", "PlaceHolder_b"]
    fused = parse_manifest(source_for(C.lora.trace(cl.f16, **C.FULL["lora"]), template="skinny",
                                      tiling=dict(WAVES_N=1, WAVES_K=2, LORA=1), split=8))
    assert [l["args"] for l in fused["launches"]] == [
        ["PlaceHolder_x", "PlaceHolder_w", "PlaceHolder_a", "PlaceHolder_b", "Partial_PACC_split", "Partial_PD_split"],
        ["Partial_PACC_combine", "Partial_PD_combine", "PlaceHolder_b", "OutputNode_0"]]


def test_chained_matmul_is_attention_marked_linear():
    g = stage_graph(C.matmul_matmul.trace(cl.f16, H=32, SQ=4096, SKV=4096, D=64))
    assert g.lowered.family == "attention" and g.lowered.problem["linear"] and g.lowered.problem["scale"] == 1.0
    assert {c.template for c in search_tiling(g, topk=100)} == {"attn_prefill"}


def test_chained_matmul_with_a_feature_major_middle_operand_is_the_same_family():
    """``(a @ b) @ c`` with ``b`` stored (K, N): the keys of the linear attention are then given
    feature-major, which the many-row kernel reads through transposing LDS reads."""
    for shapes in (dict(M=4096, N=4096, K=64), dict(M=4096, N=64, K=64)):
        prog = C.matmul_matmul_2d.trace(cl.f16, **shapes)
        g = stage_graph(prog)
        p = g.lowered.problem
        assert g.lowered.family == "attention" and p["linear"] and p["k_major"]
        assert (p["units"], p["sq"], p["skv"], p["head_dim"], p["vdim"]) == (1, 4096, shapes["N"], 64, 64)
        assert {c.template for c in search_tiling(g, topk=100)} == {"attn_prefill"}
        assert "#define CL_KT 1" in source_for(prog)
    assert not stage_graph(C.matmul_matmul.trace(cl.f16, H=2, SQ=64, SKV=64, D=64)).lowered.problem["k_major"]
    with pytest.raises(Exception, match="32-key steps|many-row"):       # 48 keys: no whole steps
        source_for(C.matmul_matmul_2d.trace(cl.f16, M=256, N=48, K=64))


def test_row_reductions_are_a_family():
    for fn, div, out_shape in ((C.rowsum, False, (4096, 1)), (C.rowsum_div, True, (4096, 4096))):
        g = stage_graph(fn.trace(cl.f16, M=4096, N=4096))
        assert g.lowered.family == "rowsum" and g.lowered.problem == {"M": 4096, "N": 4096, "div": div}
        assert g.outputs[0].shape == out_shape
        assert sorted(c.tiling["ROWS_PER_BLOCK"] for c in search_tiling(g, topk=10)) == [1, 2, 4]
        m = parse_manifest(source_for(fn.trace(cl.f16, M=4096, N=4096), template="rowsum", tiling=dict(ROWS_PER_BLOCK=4)))
        assert m["launches"][0]["grid"] == ["1024", "1", "1"] and m["launches"][0]["block"][0] == 256


def test_unrecognised_program_is_refused():
    from cleave_amd.frontend import Program

    p = Program("odd", cl.f16)
    a = p.input("a", [8, 8])
    p.output(a.exp().silu())
    with pytest.raises(LoweringRejected, match="match no kernel family"):
        stage_graph(p)


def test_split_stages_and_partial_buffers():
    g = stage_graph(C.gqa_decode_exact.trace(cl.f16, **C.FULL["c3"]))
    partial, combine = split_stages(g, 16)
    assert [o.shape for o in partial.outputs] == [(16, 256), (16, 256), (16, 256, 128)]
    assert [p.name for p in combine.placeholders] == ["PlaceHolder_PM", "PlaceHolder_PL", "PlaceHolder_PO"]
    assert partial_buffers(g.lowered, 16)[2][2] == "float32"
    with pytest.raises(LoweringRejected, match="does not divide"):
        split_stages(g, 3)
    (bundle,) = to_bundles([C.matmul.trace(M=128, N=128, K=4096).to_graph_structure()], split_factors=[8],
                           input_names=["x", "w"])
    assert [s.role for s in bundle] == ["partial", "combine"] and bundle[0].outputs[0].shape == (8, 128, 128)


def test_search_space_respects_gfx950_limits():
    from cleave_amd.arch import GFX950

    g = stage_graph(C.matmul.trace(cl.f16, M=4096, N=14336, K=4096))
    cands = search_tiling(g, topk=10_000)
    assert len(cands) > 50 and {c.template for c in cands} == {"gemm", "gemm_dma"}
    for c in cands:
        t = c.tiling
        assert t["BM"] % (16 * t["WM"]) == 0 and t["BN"] % (16 * t["WN"]) == 0 and t["BK"] in (32, 64)
        assert c.lds_bytes <= GFX950.lds_bytes and c.n_threads % 64 == 0 and c.n_threads <= 1024
        assert c.flat_graph is g
    assert [c.score for c in cands] == sorted(c.score for c in cands)
    # few rows: the weight-streaming template joins the pool
    skinny = search_tiling(stage_graph(C.rmsnorm_matmul.trace(cl.f16, **C.FULL["c2"])), topk=10_000)
    assert {"skinny", "gemm"} <= {c.template for c in skinny}
    assert search_tiling(g, topk=3, accept=lambda c: c.tiling["BM"] == 256)[0].tiling["BM"] == 256
    with pytest.raises(ScheduleRejected):
        search_tiling(stage_graph(C.gqa_decode_exact.trace(cl.f16, HQ=4, HKV=4, SQ=1, SKV=64, D=48)))


def test_emitted_signature_follows_the_naming_contract():
    prog = C.rmsnorm_matmul.trace(cl.f16, **C.FULL["c2"])
    m = parse_manifest(source_for(prog, template="skinny", tiling=dict(WAVES_N=1, WAVES_K=2)))
    assert [p["name"] for p in m["params"]] == ["PlaceHolder_x", "PlaceHolder_gamma", "PlaceHolder_w", "OutputNode_0"]
    assert m["out_idx"] == [-1] and m["launches"][0]["entry"] == "main_kernel" and m["launches"][0]["grid"][0] == "86"
    fused = parse_manifest(source_for(prog, template="skinny", tiling=dict(WAVES_N=1, WAVES_K=2), split=8))
    names = [p["name"] for p in fused["params"]]
    assert names == ["PlaceHolder_x", "PlaceHolder_gamma", "PlaceHolder_w", "Partial_PACC_split", "Partial_PACC_combine",
                     "Partial_PSS_split", "Partial_PSS_combine", "OutputNode_0"]
    assert fused["params"][4]["alias"] == "Partial_PACC_split" and fused["params"][3]["role"] == "scratch"
    assert [l["entry"] for l in fused["launches"]] == ["main_kernel", "main_kernel_combine"]
    assert fused["launches"][0]["grid"][:2] == ["86", "8"]


def test_paged_signature_matches_the_reference_operator():
    from cleave_amd.dynamic.paging import PAGED_DECODE_SLAB, CombineTiling, DenseAttention, PagingSpec, build_split_decode

    spec = PagingSpec(num_qo_heads=32, num_kv_heads=8, kind=PAGED_DECODE_SLAB, page_size=64)
    dense = DenseAttention(16, 32, 128, 256, "bfloat16", "bfloat16", waves=4)
    m = parse_manifest(HipCodeGen().gen(build_split_decode(spec, dense, 8, CombineTiling(split=8))))
    names = [p["name"] for p in m["params"] if p["role"] != "scratch"]
    assert names == ["PlaceHolder_Q", "PlaceHolder_K_CACHE", "PlaceHolder_V_CACHE", "PlaceHolder_KV_INDPTR",
                     "PlaceHolder_KV_INDICES", "PlaceHolder_KV_LAST_PAGE_LEN", "sm_scale", "OutputNode_0", "OutputNode_1"]
    by = {p["name"]: p for p in m["params"]}
    assert by["PlaceHolder_K_CACHE"]["shape"] == ["num_pages", 64, 8, 128] and by["OutputNode_1"]["dtype"] == "float32"
    assert by["Partial_PO_split"]["shape"] == [8, "batch", 32, 128] and m["dyn_dims"] == ["batch", "num_pages", "n_idx"]
    assert m["launches"][0]["grid"] == ["(batch * 8) * 1", "8", "1"]


def test_split_tail_of_the_direct_to_lds_matmul():
    """A launch whose last round fills at most half the compute units is also offered with that
    round's tiles run as two half-height workgroups each: one-dimensional grid, whole tiles first;
    refused where the row tiles are ragged or the A operand is stored K-major."""
    g = stage_graph(C.matmul.trace(cl.f16, M=4096, N=14336, K=4096))
    tails = [c for c in search_tiling(g, topk=10_000) if c.tiling.get("TAIL")]
    assert tails and all(c.template == "gemm_dma" for c in tails)
    big = next(c for c in tails if (c.tiling["BM"], c.tiling["BN"]) == (256, 256))
    assert big.tiling["TAIL"] == (16 * 56) % 256 == 128
    m = parse_manifest(HipCodeGen().gen(apply_tiling(big)))
    assert m["launches"][0]["grid"] == [str(16 * 56 + 128), "1", "1"]
    # 1024 tiles of 256 x 224 would be whole rounds; 896 + 0 tail tiles never carry the knob
    even = stage_graph(C.matmul.trace(cl.f16, M=4096, N=16384, K=4096))
    assert not [c for c in search_tiling(even, topk=10_000)
                if c.tiling.get("TAIL") and (c.tiling["BM"], c.tiling["BN"]) == (256, 256)]
    ragged = stage_graph(C.matmul.trace(cl.f16, M=4000, N=14336, K=4096))
    with pytest.raises(CodegenError, match="tail split"):
        HipCodeGen().gen(apply_tiling(TileDict("gemm_dma", "main", dict(BM=256, BN=256, BK=64, WM=4, WN=2, TAIL=8),
                                               flat_graph=ragged)))


def test_codegen_refuses_impossible_plans():
    g = stage_graph(C.matmul.trace(cl.f16, M=128, N=128, K=4096))
    with pytest.raises(CodegenError, match="multiple"):
        HipCodeGen().gen(apply_tiling(TileDict("gemm", "main", dict(BM=64, BN=64, BK=64, WM=2, WN=2), flat_graph=g,
                                               split_factor=None)).__class__(**{**apply_tiling(
                                                   TileDict("gemm", "main", dict(BM=64, BN=64, BK=64, WM=2, WN=2),
                                                            flat_graph=g)).__dict__, "problem": {**g.lowered.problem, "K": 4100}}))
    with pytest.raises(CodegenError, match="bytes of LDS"):          # 64 rows reduced over eight waves: 197 KB
        HipCodeGen().gen(apply_tiling(TileDict("skinny", "main", dict(WAVES_N=2, WAVES_K=4), flat_graph=stage_graph(
            C.rmsnorm_matmul.trace(cl.f16, M=64, N=1024, K=1024)))))
    with pytest.raises(CodegenError, match="three LDS stages"):      # three 64 KB images do not fit
        HipCodeGen().gen(apply_tiling(TileDict("gemm_dma", "main", dict(BM=256, BN=256, BK=64, WM=2, WN=4, STAGES=3), flat_graph=g)))
    with pytest.raises(CodegenError, match="no template"):
        HipCodeGen().gen(apply_tiling(TileDict("nonesuch", "main", {}, flat_graph=g)))
    # the value waves of the score-wave / value-wave MLA kernel walk their read-ahead ring in whole turns
    mla = stage_graph(C.mla_decode.trace(cl.bf16, B=2, H=64, D=512, PE=64, SKV=256))
    with pytest.raises(CodegenError, match="LDS_AHEAD"):
        HipCodeGen().gen(apply_tiling(TileDict("mla_decode", "main", dict(DUO=1, LDS_AHEAD=12), flat_graph=mla)))
    with pytest.raises(CodegenError):      # the value waves keep at least one of the nine panels
        HipCodeGen().gen(apply_tiling(TileDict("mla_decode", "main", dict(DUO=1, S_PANELS=9), flat_graph=mla)))
    m = parse_manifest(HipCodeGen().gen(apply_tiling(TileDict("mla_decode", "main", dict(DUO=1, LDS_AHEAD=4), flat_graph=mla))))
    assert m["launches"][0]["block"] == [512, 1, 1] and m["launches"][0]["grid"][0] == "2"
    with pytest.raises(CodegenError, match="manifest"):
        parse_manifest("__global__ void k() {}")


def test_tiling_keys_that_ask_for_a_measurement_switch_are_refused():
    """The shipped templates hold no probes; a DBG_ key in a tiling is an error, not a silent no-op."""
    g = stage_graph(C.gqa_decode_exact.trace(cl.f16, HQ=32, HKV=8, SQ=1, SKV=1024, D=128))
    for template, tiling in (("attn_decode", dict(WAVES=1, DBG_TIME=1)),):
        with pytest.raises(CodegenError, match="measurement switches"):
            HipCodeGen().gen(apply_tiling(TileDict(template, "main", tiling, flat_graph=g)))
    mla = stage_graph(C.mla_decode.trace(cl.bf16, B=2, H=64, D=512, PE=64, SKV=256))
    with pytest.raises(CodegenError, match="measurement switches"):
        HipCodeGen().gen(apply_tiling(TileDict("mla_decode", "main", dict(DUO=1, DBG_NODMA=1), flat_graph=mla)))
    templates = Path(C.__file__).parent / "codegen" / "templates"
    for f in templates.glob("*.hip"):
        assert "DBG_" not in f.read_text(), f.name


def test_matmul_rowsum_with_a_ragged_column_tile_is_refused_with_its_reason():
    """One set of accumulators sums every column tile of a row block, so a ragged last tile cannot be masked."""
    with pytest.raises(ScheduleRejected, match="N % 16 == 0"):
        search_tiling(stage_graph(C.matmul_rowsum.trace(cl.f16, M=255, N=264, K=128)))
    assert search_tiling(stage_graph(C.matmul_rowsum.trace(cl.f16, M=255, N=272, K=128)))


def test_few_row_units_go_to_the_streaming_kernel_unless_the_operator_has_none():
    plain = search_tiling(stage_graph(C.gqa_decode_exact.trace(cl.f16, HQ=4, HKV=2, SQ=5, SKV=300, D=128)), topk=50)
    assert {c.template for c in plain} == {"attn_decode"}
    for fn, shapes in ((C.qknorm, dict(HQ=4, HKV=2, SQ=5, SKV=300, D=128)), (C.matmul_matmul, dict(H=2, SQ=1, SKV=100, D=64))):
        normed = search_tiling(stage_graph(fn.trace(cl.f16, **shapes)), topk=50)
        assert normed and {c.template for c in normed} == {"attn_prefill"}
    with pytest.raises(ScheduleRejected, match="64-feature panels"):
        search_tiling(stage_graph(C.qknorm.trace(cl.f16, HQ=4, HKV=2, SQ=5, SKV=300, D=384)))


def test_contraction_lengths_off_the_64_wide_step():
    """K % 8 == 0 is enough unsplit (the register-staged kernel zeroes the last step's tail); a split wants
    whole steps per range; anything else is refused with the alignment rule."""
    for k in (8, 40, 96, 4104):
        cands = search_tiling(stage_graph(C.matmul.trace(cl.f16, M=100, N=64, K=k)), topk=100)
        assert cands and {c.template for c in cands} == {"gemm"}
    whole = search_tiling(stage_graph(C.matmul.trace(cl.f16, M=100, N=64, K=128)), topk=200)
    assert {"gemm", "gemm_dma"} <= {c.template for c in whole}
    part = split_stages(stage_graph(C.matmul.trace(cl.f16, M=100, N=64, K=192)), 2)[0]
    with pytest.raises(ScheduleRejected, match="16-byte chunks"):
        search_tiling(part)
    for shapes in (dict(M=100, N=64, K=100), dict(M=100, N=60, K=64)):
        with pytest.raises(ScheduleRejected, match="16-byte chunks"):
            search_tiling(stage_graph(C.matmul.trace(cl.f16, **shapes)))
    with pytest.raises(CodegenError, match="nor, unsplit, of 8"):
        source_for(C.matmul.trace(cl.f16, M=100, N=64, K=100), template="gemm", tiling=dict(BM=32, BN=32, BK=64, WM=1, WN=1))


def test_searches_that_find_nothing_say_why():
    for prog, reason in ((C.swiglu.trace(cl.f16, M=100, N=72, K=128), "N % 16 == 0"),
                         (C.swiglu.trace(cl.f16, M=100, N=128, K=96), "K % 64 == 0"),
                         (C.rowsum.trace(cl.f16, M=100, N=100), "N % 8 == 0"),
                         (C.gqa_decode_exact.trace(cl.f16, HQ=8, HKV=2, SQ=1, SKV=1000, D=160), "160/160 with 4 query rows"),
                         (C.gqa_decode_exact.trace(cl.f16, HQ=8, HKV=2, SQ=512, SKV=1000, D=96), "multiples of 64 up to 256")):
        with pytest.raises(ScheduleRejected, match=reason):
            search_tiling(stage_graph(prog))
    for rows in (512, 1):
        wide = search_tiling(stage_graph(C.gqa_decode_exact.trace(cl.f16, HQ=8, HKV=2, SQ=rows, SKV=1000, D=192)))
        assert wide and {c.template for c in wide} == {"attn_prefill"}


def test_matmul_tiles_with_fewer_load_units_than_waves_compile():
    """A 16-row tile under four waves has two 1 KiB load units for A: only two waves load it.  The
    test for that must be scalar to the compiler (the wave index out of a scalar register), or the
    tile's base address reaches the load's assembly in vector registers and the source does not
    compile: found at these shapes by a sweep of the default plan (needs the compiler, no GPU)."""
    from cleave_amd.runtime import shim
    shim.load()
    for shapes in (dict(M=336, N=1536, K=1024), dict(M=768, N=792, K=1024)):
        for fn, dtype in ((C.matmul_nt, cl.f16), (C.matmul_nt, cl.bf16)):
            source = source_for(fn.trace(dtype, **shapes))
            text = source if isinstance(source, str) else source.code
            code, _ = shim.compile_source(text, "cleave_kernel.hip", "gfx950")
            assert len(code) > 1000
    tiling = dict(BM=16, BN=64, BK=64, WM=1, WN=4)
    source = source_for(C.matmul.trace(cl.f16, M=600, N=776, K=576), template="gemm_dma", tiling=tiling)
    shim.compile_source(source if isinstance(source, str) else source.code, "cleave_kernel.hip", "gfx950")


def test_hot_kernels_keep_their_values_in_registers():
    """The graded operators' kernels as the run-time compiler builds them: no spilled register and
    no scratch memory (needs the compiler, no GPU).  A spill inside a kernel's loop costs more than
    its own traffic here, because the reload waits for every tile load in flight: the wide-key
    attention kernel ran a quarter slower for fourteen spilled address registers, and the listing
    of the offline compiler, which allocates differently, did not show them."""
    from cleave_amd.pipeline.direct import kernel_for
    from cleave_amd.runtime import shim
    shim.load()
    plans = [
        ("rmsnorm -> matmul M=16", C.CASES["c2"], C.FULL["c2"], dict(template="skinny", tiling=dict(WAVES_N=1, WAVES_K=2), split=8)),
        ("GQA decode", C.CASES["c3"], C.FULL["c3"], dict(template="attn_decode", tiling=dict(WAVES=1, SKEW=30), split=8)),
        ("MLA decode", C.CASES["c4"], C.FULL["c4"], dict(template="mla_decode", tiling=dict(DUO=1, LDS_AHEAD=4), split=8)),
        ("matmul 4096x14336x4096", C.CASES["c1"], dict(M=4096, N=14336, K=4096),
         dict(template="gemm_dma", tiling=dict(BM=256, BN=256, BK=64, WM=4, WN=2, TAIL=128))),
        ("dense attention d=64", C.CASES["c3"], dict(HQ=32, HKV=8, SQ=4096, SKV=4096, D=64),
         dict(template="attn_prefill", tiling=dict(SHARED=1))),
    ]
    kernels = [(label, kernel_for(case[0].trace(case[1], **sizes), **how)) for label, case, sizes, how in plans]
    kernels.append(("attention 192/128 wide", kernel_for(C.mla_prefill.trace(cl.f16, H=128, SQ=4096, SKV=4096, DK=192, DV=128))))
    for label, kernel in kernels:
        stages = getattr(kernel, "stages", None) or [kernel]
        for stage in stages:
            for entry in stage.stats:
                assert entry["spilled_vgprs"] == 0 and entry["scratch_bytes"] == 0, (label, entry)
                assert entry["vgprs"] <= 512 and entry["lds_bytes"] <= 160 * 1024, (label, entry)


def test_a_split_of_a_family_without_a_contraction_is_refused_with_its_reason():
    """Row reductions have nothing to split: asking for a split is a refusal that says so (it
    was a KeyError from inside the lowering)."""
    graph = stage_graph(C.rowsum_div.trace(cl.f16, M=64, N=256))
    with pytest.raises(LoweringRejected, match="no split form"):
        split_stages(graph, 4)
    with pytest.raises(LoweringRejected, match="no split form"):
        source_for(C.rowsum_div.trace(cl.f16, M=64, N=256), split=4)


def test_shipped_registry_kernels_keep_their_values_in_registers():
    """The nine registry operators' shipped kernels as the run-time compiler builds them: nothing
    spilled, no scratch memory, and the streaming decode forms within the 256 registers that let two
    waves share a SIMD (needs the compiler, no GPU)."""
    from cleave_amd.dynamic import OPERATORS
    from cleave_amd.runtime import shim
    from cleave_amd.runtime.compile import _compile, _load_main_kernel_from_code
    shim.load()
    assert len(OPERATORS) == 9
    for name, op in OPERATORS.items():
        loaded = _load_main_kernel_from_code(op.kernel_source())
        for entry in _compile(loaded, loaded.manifest["out_idx"]).stats:
            assert entry["spilled_vgprs"] == 0 and entry["scratch_bytes"] == 0, (name, entry)
            if name.startswith("gqa_paged_decode"):
                assert entry["vgprs"] <= 256, (name, entry)
