"""GPU parity of the dense attention family with many query rows per unit (the reference's
prefill-shaped end-to-end cases ``flash_attention_sd``, ``mha_bhsd``, ``gqa_bhsd``, ``mqa_bhsd``:
``tests/schedule/end2end/test_end2end.py:14-43``) through the kernel whose four waves share
every key tile: against the numpy oracle at small sizes (ragged row and key counts, head widths
64 / 128 / 256, both element types), and at the reference's sizes against a sample of rows."""

import numpy as np
import pytest
import torch

import cleave_amd.lang as cl
from cleave_amd import pipeline as P
from oracle import program_oracle
from cleave_amd import examples as C
from cleave_amd.pipeline.direct import kernel_for, stage_graph

pytestmark = pytest.mark.gpu


def _check(fn, dtype, shapes, seed=7, **how):
    prog = fn.trace(dtype, **shapes)
    args = prog.random_inputs(seed=seed)
    how = how or dict(template="attn_prefill", tiling=dict(SHARED=1))
    print(f"dense prefill case {prog.name} {dtype} {shapes} {how}", flush=True)
    out = kernel_for(prog, **how)(*args)
    torch.cuda.synchronize()
    want = program_oracle.evaluate(prog, list(args))[0]
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("shapes", [
    dict(HQ=8, HKV=2, SQ=200, SKV=300, D=64),          # GQA, ragged rows (800 per unit) and keys
    dict(HQ=4, HKV=4, SQ=130, SKV=64, D=128),          # MHA, two items per unit with a 2-row tail
    dict(HQ=8, HKV=1, SQ=40, SKV=1000, D=128),         # MQA, 320 rows on one key set
    dict(HQ=2, HKV=2, SQ=64, SKV=33, D=256),           # widest head, one full step and a 1-key tail
], ids=["gqa_d64", "mha_d128", "mqa_d128", "mha_d256"])
def test_dense_prefill_against_the_oracle(shapes):
    _check(C.gqa_decode_exact, cl.f16, shapes)


@pytest.mark.parametrize("keys", [32, 64, 96, 128, 160, 256])
def test_widest_head_with_whole_steps_of_keys(keys):
    """256-wide heads over one to eight whole 32-key steps (no masked tail).  Four steps once came
    back wrong in the first row tile of every wave: the step count is a constant in this mode, the
    compiler laid the four steps out in a straight line and, short of registers, restored a spilled
    query fragment with one register missing.  The loop's trip count is kept from the optimiser now."""
    _check(C.gqa_decode_exact, cl.f16, dict(HQ=1, HKV=1, SQ=152, SKV=keys, D=256), seed=37705)
    _check(C.gqa_decode_exact, cl.bf16, dict(HQ=4, HKV=2, SQ=40, SKV=keys, D=256), seed=3)


def test_dense_prefill_bf16_and_the_shifted_softmax_form():
    _check(C.gqa_decode_exact, cl.bf16, dict(HQ=8, HKV=2, SQ=96, SKV=257, D=128))
    _check(C.gqa_decode_shift, cl.f16, dict(HQ=8, HKV=4, SQ=100, SKV=200, D=64))


def test_key_width_differs_from_value_width():
    """192-wide keys, 128-wide values (the reference's ``mla_prefill_bhsd`` case): small against
    the oracle, then the reference's size on a sample of rows."""
    _check(C.mla_prefill, cl.f16, dict(H=4, SQ=100, SKV=150, DK=192, DV=128))
    _check(C.mla_prefill, cl.bf16, dict(H=2, SQ=64, SKV=64, DK=128, DV=64))
    shapes = dict(H=128, SQ=4096, SKV=4096, DK=192, DV=128)
    prog = C.mla_prefill.trace(cl.f16, **shapes)
    q, k, v = prog.random_inputs(seed=17)
    out = kernel_for(prog)(q, k, v)
    torch.cuda.synchronize()
    gen = np.random.default_rng(2)
    for h, s in zip(gen.integers(0, 128, 32), gen.integers(0, 4096, 32)):
        w = torch.softmax((k[h].double() @ q[h, s].double()) / 192 ** 0.5, dim=0)
        np.testing.assert_allclose(out[h, s].float().cpu().numpy(), (w @ v[h].double()).float().cpu().numpy(),
                                   rtol=1e-2, atol=1e-2)


def test_qk_norm_attention():
    """RMSNorm of queries and keys fused into the attention (the reference's ``qknorm`` case,
    (1, 64, 8, 4096, 4096, 128)): small against the oracle with both, only the keys and only the
    queries normalised; then the reference's size on a sample of rows."""
    import cleave_amd

    @cleave_amd.jit
    def k_only(q: cl.Tensor["HQ", "SQ", "D"], k: cl.Tensor["HKV", "SKV", "D"], v: cl.Tensor["HKV", "SKV", "D"]):
        return cl.softmax((q @ cl.rms_norm(k, dim=-1, eps=1e-5).mT) * 0.25, dim=-1) @ v

    @cleave_amd.jit
    def q_only(q: cl.Tensor["HQ", "SQ", "D"], k: cl.Tensor["HKV", "SKV", "D"], v: cl.Tensor["HKV", "SKV", "D"]):
        return cl.softmax((cl.rms_norm(q, dim=-1) @ k.mT) * 0.25, dim=-1) @ v

    _check(C.qknorm, cl.f16, dict(HQ=8, HKV=2, SQ=100, SKV=300, D=128))
    _check(C.qknorm, cl.bf16, dict(HQ=4, HKV=4, SQ=70, SKV=45, D=64))
    _check(k_only, cl.f16, dict(HQ=8, HKV=1, SQ=33, SKV=200, D=128))
    _check(q_only, cl.f16, dict(HQ=2, HKV=2, SQ=96, SKV=64, D=64))
    # (the keys normalised by a launch of their own ahead of the attention kernel)
    pre = dict(template="attn_prefill", tiling=dict(SHARED=1, KPRE=1))
    _check(C.qknorm, cl.f16, dict(HQ=8, HKV=2, SQ=100, SKV=300, D=128), **pre)
    _check(C.qknorm, cl.bf16, dict(HQ=4, HKV=4, SQ=70, SKV=45, D=64), **pre)
    _check(k_only, cl.f16, dict(HQ=8, HKV=1, SQ=33, SKV=200, D=128), **pre)
    _check(C.qknorm, cl.f16, dict(HQ=8, HKV=2, SQ=256, SKV=512, D=128), split=4, **pre)
    shapes = dict(HQ=64, HKV=8, SQ=4096, SKV=4096, D=128)
    prog = C.qknorm.trace(cl.f16, **shapes)
    q, k, v = prog.random_inputs(seed=19)
    norm = lambda x: x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6)   # noqa: E731
    for how in (dict(template="attn_prefill", tiling=dict(SHARED=1)), pre):
        out = kernel_for(prog, **how)(q, k, v)
        torch.cuda.synchronize()
        gen = np.random.default_rng(3)
        for h, s in zip(gen.integers(0, 64, 32), gen.integers(0, 4096, 32)):
            w = torch.softmax((norm(k[h // 8].double()) @ norm(q[h, s].double())) / 128 ** 0.5, dim=0)
            np.testing.assert_allclose(out[h, s].float().cpu().numpy(), (w @ v[h // 8].double()).float().cpu().numpy(),
                                       rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("waves", [1, 2, 4])
def test_streaming_kernel_strides_keys_and_values_by_their_own_widths(waves):
    """The streaming (decode) kernel on operands whose key width is not the value width: K rows
    are 192 or 64 elements apart, V rows 128.  (It once walked V with the key stride.)"""
    for shapes in (dict(H=3, SQ=20, SKV=150, DK=192, DV=128), dict(H=2, SQ=5, SKV=70, DK=64, DV=128)):
        prog = C.mla_prefill.trace(cl.f16, **shapes)
        args = prog.random_inputs(seed=23)
        print(f"streaming kernel, widths {shapes['DK']}/{shapes['DV']}, waves {waves}: {shapes}", flush=True)
        out = kernel_for(prog, template="attn_decode", tiling=dict(WAVES=waves))(*args)
        torch.cuda.synchronize()
        np.testing.assert_allclose(out.float().cpu().numpy(), program_oracle.evaluate(prog, list(args))[0],
                                   rtol=1e-2, atol=1e-2)


def test_chained_matmul_is_attention_without_softmax():
    """``(q @ k^T) @ v`` (the reference's ``matmul_matmul_bhsd`` case, (1, 32, 4096, 4096, 64)):
    small against the oracle (ragged rows and keys), then the reference's size on a sample of rows
    with the scores rounded to the element type as the second product's input is."""
    def scaled(prog, seed):
        q, k, v = prog.random_inputs(seed=seed)
        return (q.float() / 8).to(q.dtype), k, v            # keeps sums of thousands of products inside f16

    for dtype, shapes in ((cl.f16, dict(H=3, SQ=100, SKV=150, D=64)), (cl.bf16, dict(H=2, SQ=64, SKV=33, D=128))):
        prog = C.matmul_matmul.trace(dtype, **shapes)
        args = scaled(prog, 29)
        print(f"chained matmul case {dtype} {shapes}", flush=True)
        out = kernel_for(prog)(*args)
        torch.cuda.synchronize()
        want = program_oracle.evaluate(prog, list(args))[0]
        # the weights here are raw scores of magnitude well above 1 kept to 11 (f16) or 8 (bf16) bits, and the sums
        # cancel: the absolute tolerance follows the magnitude of the outputs and the width of the element type
        atol = 1e-2 + np.abs(want).max() * (2.0 ** -6 if dtype is cl.bf16 else 2.0 ** -9)
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=atol)
    shapes = dict(H=32, SQ=4096, SKV=4096, D=64)
    prog = C.matmul_matmul.trace(cl.f16, **shapes)
    q, k, v = scaled(prog, 31)
    out = kernel_for(prog)(q, k, v)
    torch.cuda.synchronize()
    gen = np.random.default_rng(4)
    for h, s in zip(gen.integers(0, 32, 32), gen.integers(0, 4096, 32)):
        w = (k[h].float() @ q[h, s].float()).to(torch.float16).double()
        want = (w @ v[h].double()).float().cpu().numpy()
        np.testing.assert_allclose(out[h, s].float().cpu().numpy(), want, rtol=1e-2, atol=1e-2 * max(1.0, np.abs(want).max() / 16))


def test_chained_matmul_with_a_feature_major_middle_operand():
    """``(a @ b) @ c`` with ``b`` stored (K, N): the reference's ``matmul_matmul_small_n`` (4096, 64, 64)
    and ``matmul_matmul_small_k`` (4096, 4096, 64) cases plus a small ragged-row one, each against
    the oracle (which keeps the intermediate in fp32; the kernel rounds it to the element type, so
    the absolute tolerance follows the magnitude of the outputs)."""
    for dtype, shapes, seed in ((cl.f16, dict(M=200, N=96, K=64), 41), (cl.bf16, dict(M=128, N=32, K=128), 42),
                                (cl.f16, dict(M=4096, N=64, K=64), 43), (cl.f16, dict(M=4096, N=4096, K=64), 44)):
        prog = C.matmul_matmul_2d.trace(dtype, **shapes)
        a, b, c = prog.random_inputs(seed=seed)
        a = (a.float() / 8).to(a.dtype)                       # keeps sums of thousands of products inside f16
        print(f"feature-major chained matmul case {dtype} {shapes}", flush=True)
        out = kernel_for(prog)(a, b, c)
        torch.cuda.synchronize()
        want = program_oracle.evaluate(prog, [a, b, c])[0]
        atol = 1e-2 + np.abs(want).max() * (2.0 ** -6 if dtype is cl.bf16 else 2.0 ** -9)
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=atol)
        # independent of the oracle: a sample of rows in float64 with the intermediate rounded as the kernel rounds it
        gen = np.random.default_rng(seed)
        for m in gen.integers(0, shapes["M"], 8):
            w = (a[m].float() @ b.float()).to(a.dtype).double()
            row = (w @ c.double()).float().cpu().numpy()
            np.testing.assert_allclose(out[m].float().cpu().numpy(), row, rtol=1e-2, atol=1e-2 * max(1.0, np.abs(row).max() / 16))


@pytest.mark.parametrize("split", [2, 4, 8])
def test_many_row_attention_split_over_the_keys(split):
    """Keys cut into equal ranges, one workgroup per (128 rows, range), f32 partials merged by the
    decode kernels' combine: softmax attention (reference points differ per range), key ranges
    that end inside a 32-key step, and the shifted form."""
    for fn, dtype, shapes in ((C.gqa_decode_exact, cl.f16, dict(HQ=8, HKV=2, SQ=100, SKV=320, D=64)),
                              (C.gqa_decode_exact, cl.bf16, dict(HQ=4, HKV=4, SQ=130, SKV=1000, D=128)),
                              (C.gqa_decode_shift, cl.f16, dict(HQ=8, HKV=4, SQ=64, SKV=200, D=64)),
                              (C.mla_prefill, cl.f16, dict(H=4, SQ=100, SKV=152, DK=192, DV=128))):
        prog = fn.trace(dtype, **shapes)
        args = prog.random_inputs(seed=51 + split)
        print(f"split-key many-row attention case {prog.name} {dtype} {shapes} split={split}", flush=True)
        out = kernel_for(prog, template="attn_prefill", tiling=dict(SHARED=1), split=split)(*args)
        torch.cuda.synchronize()
        want = program_oracle.evaluate(prog, list(args))[0]
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("split", [2, 8])
def test_chained_matmul_split_over_the_middle_dimension(split):
    """``(a @ b) @ c`` with the N walk cut into ranges (plain sums of f32 partials), ``b`` given
    (K, N) or as its transpose: the reference's (4096, 4096, 64) size and a small one."""
    for fn, dtype, shapes, seed in ((C.matmul_matmul_2d, cl.f16, dict(M=200, N=256, K=64), 61),
                                    (C.matmul_matmul_2d, cl.f16, dict(M=4096, N=4096, K=64), 62),
                                    (C.matmul_matmul, cl.bf16, dict(H=2, SQ=100, SKV=144, D=128), 63)):
        prog = fn.trace(dtype, **shapes)
        args = list(prog.random_inputs(seed=seed))
        args[0] = (args[0].float() / 8).to(args[0].dtype)      # keeps sums of thousands of products inside f16
        print(f"split chained matmul case {prog.name} {dtype} {shapes} split={split}", flush=True)
        out = kernel_for(prog, split=split)(*args)
        torch.cuda.synchronize()
        want = program_oracle.evaluate(prog, args)[0]
        atol = 1e-2 + np.abs(want).max() * (2.0 ** -6 if dtype is cl.bf16 else 2.0 ** -9)
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=atol)


def test_search_prefers_the_shared_kernel_for_many_rows_and_keeps_decode_for_few():
    from cleave_amd.schedule import search_tiling

    many = search_tiling(stage_graph(C.gqa_decode_exact.trace(cl.f16, HQ=32, HKV=8, SQ=4096, SKV=4096, D=64)), topk=3)
    assert many[0].template == "attn_prefill" and {c.template for c in many} == {"attn_prefill", "attn_decode"}
    few = search_tiling(stage_graph(C.gqa_decode_exact.trace(cl.f16, **C.FULL["c3"])), topk=20)
    assert {c.template for c in few} == {"attn_decode"}


@pytest.mark.parametrize("shapes", [dict(HQ=32, HKV=8, SQ=4096, SKV=4096, D=64), dict(HQ=32, HKV=32, SQ=4096, SKV=4096, D=64),
                                    dict(HQ=32, HKV=1, SQ=4096, SKV=4096, D=64), dict(HQ=1, HKV=1, SQ=4096, SKV=4096, D=64)],
                         ids=["gqa_bhsd", "mha_bhsd", "mqa_bhsd", "flash_attention_sd"])
def test_reference_end_to_end_sizes_on_a_sample_of_rows(shapes):
    """The searched best kernel at the reference's sizes; 64 query rows spread over heads and
    positions are recomputed in float64."""
    prog = C.gqa_decode_exact.trace(cl.f16, **shapes)
    q, k, v = prog.random_inputs(seed=13)
    out = kernel_for(prog)(q, k, v)
    torch.cuda.synchronize()
    gen = np.random.default_rng(1)
    group = shapes["HQ"] // shapes["HKV"]
    for h, s in zip(gen.integers(0, shapes["HQ"], 64), gen.integers(0, shapes["SQ"], 64)):
        kk, vv = k[h // group].double(), v[h // group].double()
        w = torch.softmax((kk @ q[h, s].double()) / shapes["D"] ** 0.5, dim=0)
        np.testing.assert_allclose(out[h, s].float().cpu().numpy(), (w @ vv).float().cpu().numpy(), rtol=1e-2, atol=1e-2)


def test_dense_prefill_compiles_end_to_end(cache_root):
    shapes = dict(HQ=8, HKV=2, SQ=512, SKV=512, D=128)
    kernel = P.compile(C.gqa_decode_exact, shapes=shapes, dtype=cl.f16, split=False, schedule=P.ScheduleConfig(topk=4),
                       eval=P.EvalConfig(warmup=2, iters=10, max_parallel=2))
    # (at this size the streaming kernel with four waves may still win: both forms are searched and validated)
    assert len(kernel.report.correct) == len(kernel.report) >= 2
    assert {"attn_prefill", "attn_decode"} <= {r.label.split("#")[1].split()[1].split("[")[0] for r in kernel.report.correct}
    prog = C.gqa_decode_exact.trace(cl.f16, **shapes)
    args = prog.random_inputs(seed=2)
    np.testing.assert_allclose(kernel(*args).float().cpu().numpy(), program_oracle.evaluate(prog, list(args))[0],
                               rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("rows", [1, 3, 17, 40, 63])
def test_few_row_units_of_the_operators_that_exist_in_this_kernel_only(rows):
    """QK-norm attention and the chained matmuls have no streaming (decode) form: with fewer than 64
    query rows per unit the search still hands them to the LDS-shared kernel (one workgroup per
    unit, the rest of its 128 rows masked), split over the keys or not."""
    from cleave_amd.schedule import search_tiling

    def chained(fn, shapes, **how):
        # first operand scaled and the tolerance following the outputs' magnitude, as in the chained tests above
        prog = fn.trace(cl.f16, **shapes)
        first, *rest = prog.random_inputs(seed=7)
        args = [(first.float() / 8).to(first.dtype), *rest]
        print(f"few-row chained case {prog.name} {shapes} {how}", flush=True)
        out = kernel_for(prog, **how)(*args)
        torch.cuda.synchronize()
        want = program_oracle.evaluate(prog, args)[0]
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2 + np.abs(want).max() * 2.0 ** -9)

    searched = dict(template=None)
    for shapes in (dict(HQ=4, HKV=2, SQ=rows, SKV=300, D=128), dict(HQ=2, HKV=2, SQ=rows, SKV=64, D=64)):
        assert search_tiling(stage_graph(C.qknorm.trace(cl.f16, **shapes)))[0].template == "attn_prefill"
        _check(C.qknorm, cl.f16, shapes, **searched)
        _check(C.qknorm, cl.f16, shapes, split=4, **searched)
    shapes = dict(H=2, SQ=rows, SKV=100, D=64)
    assert search_tiling(stage_graph(C.matmul_matmul.trace(cl.f16, **shapes)))[0].template == "attn_prefill"
    chained(C.matmul_matmul, shapes)
    chained(C.matmul_matmul, shapes, split=4)
    chained(C.matmul_matmul_2d, dict(M=rows, N=96, K=64))


def test_widths_only_the_many_row_kernel_takes():
    """192-wide keys and values: the streaming kernel has no form for a 192-wide value (64 or a
    multiple of 128), the LDS-shared kernel works in 64-feature panels; the search hands it over."""
    from cleave_amd.schedule import search_tiling

    shapes = dict(HQ=4, HKV=2, SQ=100, SKV=300, D=192)
    assert {c.template for c in search_tiling(stage_graph(C.gqa_decode_exact.trace(cl.f16, **shapes)))} == {"attn_prefill"}
    _check(C.gqa_decode_exact, cl.f16, shapes, template=None)
    _check(C.gqa_decode_exact, cl.bf16, dict(HQ=2, HKV=2, SQ=64, SKV=512, D=192), template=None, split=4)
    _check(C.gqa_decode_shift, cl.f16, dict(HQ=8, HKV=1, SQ=70, SKV=77, D=192), template=None)
    # decode-shaped units of that width have no other kernel either
    _check(C.gqa_decode_exact, cl.f16, dict(HQ=8, HKV=2, SQ=1, SKV=1000, D=192), template=None)
    _check(C.gqa_decode_exact, cl.f16, dict(HQ=8, HKV=2, SQ=3, SKV=1024, D=192), template=None, split=8)


def test_rising_maximum_in_the_many_row_kernel():
    """Scores that grow along the key axis: every row's softmax reference point is raised several times
    on the way (the cold path of the kernel whose waves share the key tiles: a ballot, a maximum over the
    key groups, sums and accumulators rescaled by a factor strictly between 0 and 1), unsplit and split over
    the keys, 64 and 128 wide."""
    for d, split in ((64, None), (128, None), (128, 4), (64, 2)):
        shapes = dict(HQ=8, HKV=2, SQ=160, SKV=1536, D=d)
        prog = C.gqa_decode_exact.trace(cl.f16, **shapes)
        q, k, v = [t.cpu() for t in prog.random_inputs(seed=23)]
        # feature 0 of every query is 4 and feature 0 of the keys climbs with the position: every row's scaled
        # scores climb by about 35 (log2 domain) over the keys, in steps far below the raise threshold
        q[..., 0] = 4.0
        k[..., 0] = torch.linspace(0.0, 35.0 * d ** 0.5 / (4 * 1.4427), shapes["SKV"]).reshape(1, -1).to(k.dtype)
        scores = (q.float().reshape(2, 640, d) @ k.float().mT) / d ** 0.5 * 1.4427
        climbs = scores[..., -32:].mean(-1) - scores[..., :32].mean(-1)
        want = program_oracle.evaluate(prog, [q, k, v])[0]
        how = dict(template="attn_prefill", tiling=dict(SHARED=1), split=split)
        print(f"dense prefill rising maximum d={d} split={split}: mean climb {float(climbs.abs().mean()):.1f} (log2)", flush=True)
        assert float(climbs.min()) > 24.0
        out = kernel_for(prog, **how)(q.cuda(), k.cuda(), v.cuda())
        torch.cuda.synchronize()
        np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=1e-2, atol=1e-2)
