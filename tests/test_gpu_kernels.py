"""GPU parity: every template against the numpy oracle on the same seeded inputs.

Tolerance: rtol 1e-2 / atol 1e-2 against the fp32-accumulated oracle for f16/bf16 outputs.
"""

import numpy as np
import pytest
import torch

import cleave_amd
import cleave_amd.lang as cl
from oracle import program_oracle as po
from cleave_amd import examples as C
from cleave_amd.pipeline.direct import kernel_for

pytestmark = pytest.mark.gpu
RTOL = ATOL = 1e-2


def _check(program, make_inputs, shapes, **kw):
    ins = make_inputs(shapes, device="cpu")
    want = po.evaluate(program, ins)[0]
    kernel = kernel_for(program, **kw)
    print(f"case {program.name} {shapes} {kw}", flush=True)
    got = kernel(*[t.cuda() for t in ins])
    torch.cuda.synchronize()
    got = got.float().cpu().numpy().reshape(want.shape)
    np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


GEMM_TILES = [dict(BM=32, BN=32, BK=64, WM=1, WN=1), dict(BM=64, BN=64, BK=64, WM=2, WN=2),
              dict(BM=128, BN=128, BK=64, WM=2, WN=2),
              # one 16-row operand tile per wave along M (and along both axes)
              dict(BM=16, BN=32, BK=64, WM=1, WN=2, GDEPTH=2), dict(BM=16, BN=16, BK=64, WM=1, WN=1, GDEPTH=1),
              dict(BM=32, BN=32, BK=64, WM=2, WN=2, GDEPTH=2), dict(BM=16, BN=64, BK=64, WM=1, WN=1)]


@pytest.mark.parametrize("tiling", GEMM_TILES, ids=lambda t: "x".join(str(v) for v in t.values()))
@pytest.mark.parametrize("split", [None, 4])
def test_matmul_gemm_small(tiling, split):
    fn, dt, mk = C.CASES["c1"]
    shapes = dict(M=96, N=136, K=512)
    _check(fn.trace(dt, **shapes), mk, shapes, template="gemm", tiling=tiling, split=split)


@pytest.mark.parametrize("tiling", [dict(BM=256, BN=256, BK=64, WM=2, WN=4, GDEPTH=1),
                                    dict(BM=256, BN=128, BK=64, WM=4, WN=2, GDEPTH=2, GROUP_M=2),
                                    dict(BM=128, BN=128, BK=64, WM=2, WN=2, GDEPTH=1, GROUP_M=3)],
                         ids=lambda t: "x".join(str(v) for v in t.values()))
def test_matmul_gemm_large_tiles(tiling):
    """Ragged tile counts (3 x 4 or 5 x 7 tiles, not multiples of the XCD count or of GROUP_M)
    exercise the workgroup renumbering and the clamped edge loads; K gives an odd step count."""
    fn, dt, mk = C.CASES["c1"]
    shapes = dict(M=600, N=776, K=448)
    _check(fn.trace(dt, **shapes), mk, shapes, template="gemm", tiling=tiling)


DMA_TILES = [dict(BM=16, BN=16, BK=64, WM=1, WN=1), dict(BM=32, BN=64, BK=64, WM=1, WN=2),
             dict(BM=64, BN=64, BK=64, WM=2, WN=2), dict(BM=128, BN=128, BK=64, WM=2, WN=2),
             dict(BM=256, BN=128, BK=64, WM=4, WN=2), dict(BM=128, BN=256, BK=64, WM=2, WN=4, GROUP_M=2),
             dict(BM=256, BN=256, BK=64, WM=2, WN=2),
             dict(BM=16, BN=64, BK=64, WM=1, WN=4)]             # fewer load units for A than waves


@pytest.mark.parametrize("tiling", DMA_TILES, ids=lambda t: "x".join(str(v) for v in t.values()))
@pytest.mark.parametrize("split", [None, 3])
def test_matmul_gemm_dma(tiling, split):
    """Direct-to-LDS matmul: ragged tile counts on both axes (edge rows and column chunks are
    clamped), an odd number of K steps per split (the two-stage loop ends on either stage)."""
    fn, dt, mk = C.CASES["c1"]
    shapes = dict(M=600, N=776, K=576)
    _check(fn.trace(dt, **shapes), mk, shapes, template="gemm_dma", tiling=tiling, split=split)


@pytest.mark.parametrize("k", [64, 128, 192, 256, 448, 576])
@pytest.mark.parametrize("tiling", [dict(BM=64, BN=64, BK=64, WM=2, WN=2, STAGES=3), dict(BM=256, BN=128, BK=64, WM=4, WN=2, STAGES=3),
                                    dict(BM=128, BN=256, BK=64, WM=2, WN=4, STAGES=3, GROUP_M=2)],
                         ids=lambda t: "x".join(str(v) for v in t.values()))
def test_matmul_gemm_dma_three_stages(tiling, k):
    """Three LDS stages (loads asked for two steps ahead, spread over a step's rows, the kernel
    counting its own loads in flight): one to nine K steps, so that the walk ends on each of the
    three stages and the clamped loads past the last step land in an idle one; ragged tiles on both
    axes; split over K (three steps per split) and the transposed-weight, bf16 form as well."""
    fn, dt, mk = C.CASES["c1"]
    shapes = dict(M=600, N=776, K=k)
    _check(fn.trace(dt, **shapes), mk, shapes, template="gemm_dma", tiling=tiling)
    if k == 576:
        _check(fn.trace(dt, **shapes), mk, shapes, template="gemm_dma", tiling=tiling, split=3)
        prog = matmul_nt.trace(cl.bf16, **shapes)
        g = torch.Generator(device="cpu").manual_seed(5)
        ins = [((torch.rand(*shp, generator=g) * 2 - 1) / 24).to(torch.bfloat16) for shp in ((600, 576), (776, 576))]
        want = po.evaluate(prog, ins)[0]
        kernel = kernel_for(prog, template="gemm_dma", tiling=tiling)
        print(f"case matmul_nt bf16 gemm_dma {tiling}", flush=True)
        got = kernel(*[t.cuda() for t in ins]).float().cpu().numpy().reshape(want.shape)
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("tiling", [dict(BM=64, BN=64, BK=64, WM=2, WN=2, TAIL=24), dict(BM=64, BN=64, BK=64, WM=2, WN=2, TAIL=5),
                                    dict(BM=256, BN=128, BK=64, WM=4, WN=2, TAIL=6),
                                    dict(BM=256, BN=256, BK=64, WM=2, WN=2, TAIL=8),
                                    dict(BM=128, BN=128, BK=64, WM=2, WN=2, TAIL=28, ASM_MFMA=1)],
                         ids=lambda t: "x".join(str(v) for v in t.values()))
def test_matmul_gemm_dma_split_tail(tiling):
    """The last tiles of the launch run as two half-height workgroups each (both orders of the
    tail workgroups: halves of a tile on one XCD when the tail is a multiple of eight, neighbours
    otherwise); ragged columns; the matrix op as builtin and as assembly."""
    fn, dt, mk = C.CASES["c1"]
    shapes = dict(M=512, N=776, K=576)
    _check(fn.trace(dt, **shapes), mk, shapes, template="gemm_dma", tiling=tiling)
    if tiling["BM"] == 64:
        prog = matmul_nt.trace(cl.bf16, **shapes)
        g = torch.Generator(device="cpu").manual_seed(5)
        ins = [((torch.rand(*shp, generator=g) * 2 - 1) / 24).to(torch.bfloat16) for shp in ((512, 576), (776, 576))]
        want = po.evaluate(prog, ins)[0]
        for asm in (0, 1):
            kernel = kernel_for(prog, template="gemm_dma", tiling=dict(tiling, ASM_MFMA=asm))
            print(f"case matmul_nt bf16 gemm_dma {tiling} asm={asm}", flush=True)
            got = kernel(*[t.cuda() for t in ins]).float().cpu().numpy().reshape(want.shape)
            np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


def test_matmul_gemm_dma_bf16():
    shapes = dict(M=192, N=256, K=384)
    prog = C.matmul.trace(cl.bf16, **shapes)
    ins = [t.to(torch.bfloat16) for t in C.inputs_c1(shapes, seed=7)]
    want = po.evaluate(prog, ins)[0]
    for tiling, split in ((dict(BM=64, BN=128, BK=64, WM=2, WN=2), None), (dict(BM=32, BN=64, BK=64, WM=1, WN=2), 2)):
        kernel = kernel_for(prog, template="gemm_dma", tiling=tiling, split=split)
        print(f"case matmul bf16 gemm_dma {tiling} split={split}", flush=True)
        got = kernel(*[t.cuda() for t in ins]).float().cpu().numpy().reshape(want.shape)
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@cleave_amd.jit
def matmul_nt(x: cl.Tensor["M", "K"], w: cl.Tensor["N", "K"]):
    return x @ w.mT


@cleave_amd.jit
def matmul_tn(x: cl.Tensor["K", "M"], w: cl.Tensor["K", "N"]):
    return x.mT @ w


@pytest.mark.parametrize("template,tiling", [("gemm_dma", dict(BM=64, BN=64, BK=64, WM=2, WN=2)),
                                             ("gemm_dma", dict(BM=128, BN=256, BK=64, WM=2, WN=4)),
                                             ("gemm", dict(BM=64, BN=64, BK=64, WM=2, WN=2))],
                         ids=["dma64", "dma128x256", "staged64"])
def test_matmul_transposed_operands(template, tiling):
    """B stored (N, K) (both operands K-minor) and A stored (K, M) (both K-major): the other two
    combinations of the 16-byte and the transposing fragment readers."""
    g = torch.Generator(device="cpu").manual_seed(11)
    M, N, K = 200, 328, 320
    for fn, shapes_in in ((matmul_nt, ((M, K), (N, K))), (matmul_tn, ((K, M), (K, N)))):
        prog = fn.trace(cl.f16, M=M, N=N, K=K)
        ins = [((torch.rand(*shp, generator=g) * 2 - 1) / K ** 0.5).to(torch.float16) for shp in shapes_in]
        want = po.evaluate(prog, ins)[0]
        kernel = kernel_for(prog, template=template, tiling=tiling)
        print(f"case {prog.name} {template} {tiling}", flush=True)
        got = kernel(*[t.cuda() for t in ins]).float().cpu().numpy().reshape(want.shape)
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("split", [None, 4, 8, 16])
def test_matmul_c1_full(split):
    fn, dt, mk = C.CASES["c1"]
    _check(fn.trace(dt, **C.FULL["c1"]), mk, C.FULL["c1"], template="gemm",
           tiling=dict(BM=64, BN=64, BK=64, WM=2, WN=2), split=split)


@pytest.mark.parametrize("tiling", [dict(WAVES_N=1, WAVES_K=1), dict(WAVES_N=2, WAVES_K=2), dict(WAVES_N=1, WAVES_K=4)],
                         ids=lambda t: "x".join(str(v) for v in t.values()))
@pytest.mark.parametrize("split", [None, 2])
def test_rmsnorm_matmul_skinny_small(tiling, split):
    fn, dt, mk = C.CASES["c2"]
    shapes = dict(M=16, K=512, N=392)     # N not a multiple of 128: the last slab is masked
    _check(fn.trace(dt, **shapes), mk, shapes, template="skinny", tiling=tiling, split=split)


@pytest.mark.parametrize("m", [1, 5, 16, 33])
def test_skinny_row_counts(m):
    fn, dt, mk = C.CASES["c2"]
    shapes = dict(M=m, K=256, N=256)
    _check(fn.trace(dt, **shapes), mk, shapes, template="skinny", tiling=dict(WAVES_N=1, WAVES_K=2))


@pytest.mark.parametrize("split", [None, 4, 8, 16])
def test_rmsnorm_matmul_c2_full(split):
    fn, dt, mk = C.CASES["c2"]
    _check(fn.trace(dt, **C.FULL["c2"]), mk, C.FULL["c2"], template="skinny",
           tiling=dict(WAVES_N=1, WAVES_K=4), split=split)


def test_rmsnorm_matmul_gemm_path():
    fn, dt, mk = C.CASES["c2"]
    shapes = dict(M=128, K=512, N=256)
    _check(fn.trace(dt, **shapes), mk, shapes, template="gemm", tiling=dict(BM=64, BN=64, BK=64, WM=2, WN=2))
    _check(fn.trace(dt, **shapes), mk, shapes, template="gemm", tiling=dict(BM=64, BN=64, BK=64, WM=2, WN=2), split=4)


@pytest.mark.parametrize("template,tiling", [("gemm", dict(BM=64, BN=64, BK=64, WM=2, WN=2)),
                                             ("gemm_dma", dict(BM=64, BN=64, BK=64, WM=2, WN=2)),
                                             ("gemm_dma", dict(BM=32, BN=64, BK=64, WM=1, WN=2))])
@pytest.mark.parametrize("split", [None, 4])
def test_batched_matmul_split_k(template, tiling, split):
    """A batch of products, unsplit and split over K into four partial products summed by the
    combine kernel: the reference's ``batched_matmul_splitk_partial`` / ``_combine`` pair at its
    size (2 entries of 128 x 128 x 4096, ``tests/schedule/end2end/test_end2end.py:15-16``), a ragged
    one, and one whose second operand is shared by pairs of entries of the first."""
    for shapes in (dict(BX=2, BW=2, M=128, N=128, K=4096), dict(BX=3, BW=3, M=72, N=136, K=512),
                   dict(BX=4, BW=2, M=64, N=128, K=1024)):
        _check(C.batched_matmul.trace(cl.f16, **shapes), C.inputs_batched, shapes, template=template, tiling=tiling,
               split=split)


@pytest.mark.parametrize("dtype", [cl.f16, cl.bf16], ids=["f16", "bf16"])
@pytest.mark.parametrize("tiling", [dict(BM=64, BN=64, BK=64, WM=2, WN=2), dict(BM=128, BN=64, BK=64, WM=4, WN=1),
                                    dict(BM=16, BN=32, BK=64, WM=1, WN=2), dict(BM=256, BN=128, BK=64, WM=4, WN=2)],
                         ids=lambda t: "x".join(str(v) for v in t.values()))
def test_rmsnorm_matmul_without_weight_on_the_direct_to_lds_matmul(dtype, tiling):
    """RMSNorm (no learned weight; with and without an epsilon) fused into the direct-to-LDS matmul
    as a scale of the product's rows: ragged tile counts on both axes, an odd number of K steps."""
    shapes = dict(M=200, N=136, K=320)
    for fn in (C.rmsnorm_matmul_plain, C.rmsnorm_matmul_eps):
        prog = fn.trace(dtype, **shapes)
        ins = [t.to(dtype.torch) for t in C.inputs_plain_norm(shapes)]
        want = po.evaluate(prog, ins)[0]
        print(f"case {prog.name} {dtype} {shapes} {tiling}", flush=True)
        got = kernel_for(prog, template="gemm_dma", tiling=tiling)(*[t.cuda() for t in ins])
        torch.cuda.synchronize()
        tol = 2e-2 if dtype is cl.bf16 else ATOL          # bf16 outputs of magnitude ~1 carry 8 bits
        np.testing.assert_allclose(got.float().cpu().numpy(), want, rtol=tol, atol=tol)


def test_rmsnorm_matmul_at_the_large_fused_shape():
    """RMSNorm -> matmul with many rows, 4096 x 6144 x 4096 (the reference's ``rmsnorm_matmul`` case,
    ``tests/schedule/end2end/test_end2end.py:37``: no weight, no epsilon), through the register-staged
    matmul that applies the norm to the A tile on its way into LDS; whole output against the oracle,
    then a sample of rows recomputed in float64 independently of it."""
    shapes = dict(M=4096, N=6144, K=4096)
    prog = C.rmsnorm_matmul_plain.trace(cl.f16, **shapes)
    x, w = C.inputs_plain_norm(shapes)
    want = po.evaluate(prog, [x, w])[0]
    for template, tiling in (("gemm", dict(BM=128, BN=128, BK=64, WM=2, WN=2)), ("gemm", dict(BM=256, BN=128, BK=64, WM=4, WN=2)),
                             ("gemm_dma", dict(BM=256, BN=256, BK=64, WM=4, WN=2)),
                             ("gemm_dma", dict(BM=256, BN=256, BK=64, WM=4, WN=2, TAIL=128))):
        print(f"case rmsnorm_matmul_plain {shapes} {template} {tiling}", flush=True)
        got = kernel_for(prog, template=template, tiling=tiling)(x.cuda(), w.cuda())
        torch.cuda.synchronize()
        got = got.float().cpu().numpy()
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)
        gen = np.random.default_rng(7)
        for m in gen.integers(0, shapes["M"], 6):
            row = x[m].double()
            ref = ((row / torch.sqrt((row * row).mean())) @ w.double()).numpy()
            np.testing.assert_allclose(got[m], ref, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("waves", [1, 2, 4])
@pytest.mark.parametrize("split", [None, 2, 8])
def test_gqa_decode_small(waves, split):
    fn, dt, mk = C.CASES["c3"]
    shapes = dict(HQ=8, HKV=2, SQ=1, SKV=416, D=128)   # 13 steps: ragged over waves and splits
    _check(fn.trace(dt, **shapes), mk, shapes, template="attn_decode", tiling=dict(WAVES=waves), split=split)


def test_gqa_decode_ragged_tail_and_shift_program():
    shapes = dict(HQ=8, HKV=2, SQ=1, SKV=200, D=128)   # 200 = 6 steps + 8 tokens
    _check(C.gqa_decode_shift.trace(C.cl.f16, **shapes), C.inputs_c3, shapes, template="attn_decode",
           tiling=dict(WAVES=2), split=None)


def test_gqa_decode_many_rows():
    shapes = dict(HQ=12, HKV=2, SQ=5, SKV=160, D=128)  # 30 rows per kv head: two row tiles
    _check(C.gqa_decode_exact.trace(C.cl.f16, **shapes), C.inputs_c3, shapes, template="attn_decode",
           tiling=dict(WAVES=2), split=2)


@pytest.mark.parametrize("split", [8, 16, 32])
def test_gqa_decode_c3_full(split):
    fn, dt, mk = C.CASES["c3"]
    _check(fn.trace(dt, **C.FULL["c3"]), mk, C.FULL["c3"], template="attn_decode", tiling=dict(WAVES=4), split=split)


@pytest.mark.parametrize("tiling,split", [(dict(WAVES=1, SKEW=30), 8), (dict(WAVES=1, SKEW=60), 8), (dict(WAVES=1, SKEW=30), 16),
                                          (dict(WAVES=2, SKEW=500), 8), (dict(WAVES=1, PREFETCH=2, SKEW=30), 32),
                                          (dict(WAVES=1, PREFETCH=3), 8)],
                         ids=lambda v: "x".join(f"{k}{x}" for k, x in v.items()) if isinstance(v, dict) else str(v))
def test_gqa_decode_c3_full_with_ranges_skewed_between_xcds(tiling, split):
    """The plans the search ranks first: a unit's splits rotated over the XCDs and the split ranges
    skewed (3 %, 6 %, and all of a pair's steps to one of its two splits), deeper load rings."""
    fn, dt, mk = C.CASES["c3"]
    _check(fn.trace(dt, **C.FULL["c3"]), mk, C.FULL["c3"], template="attn_decode", tiling=tiling, split=split)


@pytest.mark.parametrize("skv", [48, 432, 1008, 2064])
def test_gqa_decode_skewed_ranges_own_every_step_once(skv):
    """Key counts that leave pairs of splits with an odd number of steps, a single step, or none; 16 units so
    that the grid is whole groups of eight; every prefetch depth's straight-line tail."""
    shapes = dict(HQ=64, HKV=16, SQ=1, SKV=skv, D=128)
    prog = C.gqa_decode_exact.trace(C.cl.f16, **shapes)
    for tiling, split in ((dict(WAVES=1, SKEW=30), 2), (dict(WAVES=1, SKEW=250), 4), (dict(WAVES=2, SKEW=60), 8),
                          (dict(WAVES=1, PREFETCH=2, SKEW=100), 4), (dict(WAVES=1, PREFETCH=3, SKEW=500), 6)):
        _check(prog, C.inputs_c3, shapes, template="attn_decode", tiling=tiling, split=split)


def test_gqa_decode_rising_maximum():
    """Scores that grow along the KV axis raise every row's softmax reference point several times inside a
    split (the cold path: a ballot, a cross-lane maximum, a rescale of sums and accumulators with a factor
    strictly between 0 and 1), in every form of the streaming kernel: one to eight waves, split and
    unsplit, skewed ranges, deeper rings."""
    shapes = dict(HQ=64, HKV=16, SQ=1, SKV=1536, D=128)
    prog = C.gqa_decode_exact.trace(C.cl.f16, **shapes)
    q, k, v = C.inputs_c3(shapes, device="cpu")
    # k gains a component along q's direction that grows with the position: the scaled scores climb by
    # ~35 (log2 domain) over the keys, in steps far smaller than the raise threshold
    ramp = torch.linspace(0.0, 48.0, shapes["SKV"]).reshape(1, -1, 1)
    qdir = q.float().reshape(16, 4, 1, 128).mean(1)
    k = (k.float() * 0.3 + ramp * qdir / qdir.norm(dim=-1, keepdim=True)).to(k.dtype)
    ins = [q, k, v]
    want = po.evaluate(prog, ins)[0]
    spread = (q.float().reshape(16, 4, 128) @ k.float().mT / 128 ** 0.5)
    assert float((spread[..., -1] - spread[..., 0]).abs().mean()) * 1.4427 > 3 * 8, "the ramp must pass the raise threshold often"
    for tiling, split in ((dict(WAVES=1), None), (dict(WAVES=4), None), (dict(WAVES=8), 2), (dict(WAVES=1, SKEW=60), 4),
                          (dict(WAVES=2, PREFETCH=2), 2), (dict(WAVES=1, PREFETCH=3), None)):
        kernel = kernel_for(prog, template="attn_decode", tiling=tiling, split=split)
        print(f"case gqa rising maximum {tiling} split={split}", flush=True)
        got = kernel(*[t.cuda() for t in ins]).float().cpu().numpy().reshape(want.shape)
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("split", [None, 2])
def test_mla_decode_small(split):
    fn, dt, mk = C.CASES["c4"]
    _check(fn.trace(dt, **C.SMALL["c4"]), mk, C.SMALL["c4"], template="mla_decode", tiling=dict(WAVES=1), split=split)
    shapes = dict(B=2, H=64, D=512, PE=64, SKV=160)
    _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(WAVES=4), split=split)
    _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(WAVES=2, HG=2), split=split)
    _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(WAVES=1, HG=2), split=split)
    _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(WAVES=4, HG=2, VSPLIT=2), split=split)
    _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(WAVES=2, HG=1, VSPLIT=2, STAGES=2),
           split=split)


def test_mla_decode_rising_maximum():
    """Scores that keep growing along the KV axis force the running maximum up in steps of
    more than 8 (log2 domain) several times per split: the deferred rescale must stay exact."""
    fn, dt, mk = C.CASES["c4"]
    shapes = dict(B=1, H=32, D=512, PE=64, SKV=512)
    prog = fn.trace(dt, **shapes)
    q, kv, q_pe, k_pe = mk(shapes, device="cpu")
    ramp = torch.linspace(0.2, 6.0, shapes["SKV"]).reshape(1, -1, 1)
    kv = (kv.float() * 0.2 + ramp * torch.sign(q.float().mean(dim=(1,), keepdim=True))).to(kv.dtype)
    ins = [q, kv, q_pe, k_pe]
    want = po.evaluate(prog, ins)[0]
    for tiling, split in ((dict(WAVES=2, HG=1), None), (dict(WAVES=1, HG=2), 2), (dict(WAVES=2, HG=2, VSPLIT=2), 2)):
        kernel = kernel_for(prog, template="mla_decode", tiling=tiling, split=split)
        print(f"case mla rising maximum {tiling} split={split}", flush=True)
        got = kernel(*[t.cuda() for t in ins]).float().cpu().numpy().reshape(want.shape)
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("tiling,split", [(dict(WAVES=4, HG=1), 8), (dict(WAVES=4, HG=1, STAGES=4), 16),
                                          (dict(WAVES=2, HG=1, STAGES=2), 4), (dict(WAVES=4, HG=2, VSPLIT=2), 8),
                                          (dict(WAVES=8, HG=1), 16)],
                         ids=lambda v: "x".join(str(x) for x in v.values()) if isinstance(v, dict) else str(v))
def test_mla_decode_c4_full(tiling, split):
    fn, dt, mk = C.CASES["c4"]
    _check(fn.trace(dt, **C.FULL["c4"]), mk, C.FULL["c4"], template="mla_decode", tiling=tiling, split=split)


@pytest.mark.parametrize("split", [None, 2, 3, 8])
def test_mla_decode_paired_waves_small(split):
    """The score-wave / value-wave form: 64 and 128 heads, key counts that leave a ragged last step
    (a token half with every token masked among them), a single step, more splits than steps
    (empty splits), unsplit."""
    fn, dt, mk = C.CASES["c4"]
    for shapes in (dict(B=2, H=64, D=512, PE=64, SKV=192), dict(B=1, H=128, D=512, PE=64, SKV=120),
                   dict(B=3, H=64, D=512, PE=64, SKV=48), dict(B=1, H=64, D=256, PE=64, SKV=456)):
        _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(DUO=1), split=split)


@pytest.mark.parametrize("split", [None, 2, 3, 8])
def test_mla_decode_paired_waves_with_shared_loading(split):
    """The same cases with the score waves asking for part of every image's panels (from the
    third image on): one, about half, and all but one of them; one to twelve steps per split, so
    that splits end before, at and after the first shared image."""
    fn, dt, mk = C.CASES["c4"]
    for shapes, panels in ((dict(B=2, H=64, D=512, PE=64, SKV=192), 4), (dict(B=1, H=128, D=512, PE=64, SKV=120), 1),
                           (dict(B=3, H=64, D=512, PE=64, SKV=48), 8), (dict(B=1, H=64, D=256, PE=64, SKV=456), 2),
                           (dict(B=1, H=64, D=512, PE=64, SKV=384), 4)):
        _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(DUO=1, LDS_AHEAD=4, S_PANELS=panels),
               split=split)


def test_mla_decode_paired_waves_rising_maximum():
    """Scores that keep growing along the KV axis: the score waves raise their reference points
    several times per split, each token half on its own, and the value waves must rescale
    accumulators, sums and the lower half's weights at exactly those steps."""
    fn, dt, mk = C.CASES["c4"]
    shapes = dict(B=1, H=64, D=512, PE=64, SKV=512)
    prog = fn.trace(dt, **shapes)
    q, kv, q_pe, k_pe = mk(shapes, device="cpu")
    ramp = torch.linspace(0.2, 6.0, shapes["SKV"]).reshape(1, -1, 1)
    kv = (kv.float() * 0.2 + ramp * torch.sign(q.float().mean(dim=(1,), keepdim=True))).to(kv.dtype)
    ins = [q, kv, q_pe, k_pe]
    want = po.evaluate(prog, ins)[0]
    for split, tiling in ((None, dict(DUO=1)), (2, dict(DUO=1)), (4, dict(DUO=1)), (2, dict(DUO=1, LDS_AHEAD=4, S_PANELS=4))):
        kernel = kernel_for(prog, template="mla_decode", tiling=tiling, split=split)
        print(f"case mla paired waves rising maximum split={split} {tiling}", flush=True)
        got = kernel(*[t.cuda() for t in ins]).float().cpu().numpy().reshape(want.shape)
        np.testing.assert_allclose(got, want, rtol=RTOL, atol=ATOL)


def test_mla_decode_paired_waves_read_ahead_depths():
    """The value waves' operand ring at its other depths (2, 4 and 16 feature blocks read ahead, across
    the barrier at the end of every step)."""
    fn, dt, mk = C.CASES["c4"]
    shapes = dict(B=2, H=64, D=512, PE=64, SKV=328)
    for ahead in (4, 8, 32):
        _check(fn.trace(dt, **shapes), mk, shapes, template="mla_decode", tiling=dict(DUO=1, LDS_AHEAD=ahead), split=2)


@pytest.mark.parametrize("split", [4, 8, 16])
@pytest.mark.parametrize("tiling", [dict(DUO=1), dict(DUO=1, LDS_AHEAD=4, S_PANELS=4)], ids=["value-waves-load", "shared-loading"])
def test_mla_decode_paired_waves_c4_full(tiling, split):
    fn, dt, mk = C.CASES["c4"]
    _check(fn.trace(dt, **C.FULL["c4"]), mk, C.FULL["c4"], template="mla_decode", tiling=tiling, split=split)


def test_graph_replay_timer_matches_eager_results_and_time():
    """The graph-replay timer (a fused partial + combine pair captured ``graph_batch`` times):
    every replayed batch must leave the eager result in the output, with the program's own eager
    launches and synchronisations between the timings, and both timers must agree on the time."""
    fn, dt, mk = C.CASES["c2"]
    shapes = C.FULL["c2"]
    prog = fn.trace(dt, **shapes)
    kernel = kernel_for(prog, template="skinny", tiling=dict(WAVES_N=1, WAVES_K=4), split=4)
    args = [t.cuda() for t in mk(shapes, device="cpu")]
    other = [t.cuda() for t in mk(shapes, seed=7)]
    want = kernel(*args).clone()
    torch.cuda.synchronize()
    eager_ms = kernel.time(*args, warmup=3, iters=50)
    times = []
    for r in range(4):
        print(f"case graph timer replay {r}", flush=True)
        ms = kernel.time(*args, warmup=1, iters=60, graph_batch=20, rotate=[other] if r % 2 else None)
        times.append(ms)
        torch.cuda.synchronize()
        assert torch.equal(kernel.last_timed_outputs[0], want)
        assert torch.equal(kernel(*args), want)            # eager work between the replays
    assert all(0 < t < 5 * eager_ms for t in times) and min(times) < 1.5 * eager_ms


@pytest.mark.parametrize("k", [8, 40, 72, 96, 200, 1000, 4104])
def test_matmul_with_a_ragged_last_k_step(k):
    """K a multiple of 8 but not of the 64-wide step: the register-staged kernel zeroes the chunks
    past K on their way to LDS.  Row-major and both transposed layouts (each loader form), both
    prefetch depths, tiles with whole and half transposed blocks, the searched best plan, a batched
    product and the fused RMSNorm (with and without the learned weight)."""
    fn, dt, mk = C.CASES["c1"]
    shapes = dict(M=100, N=136, K=k)
    for tiling in (dict(BM=32, BN=32, BK=64, WM=1, WN=1), dict(BM=64, BN=64, BK=64, WM=2, WN=2, GDEPTH=2),
                   dict(BM=16, BN=128, BK=64, WM=1, WN=4)):
        _check(fn.trace(dt, **shapes), mk, shapes, template="gemm", tiling=tiling)
    _check(fn.trace(dt, **shapes), mk, shapes)
    g = torch.Generator(device="cpu").manual_seed(k)
    for prog, dims in ((matmul_nt.trace(cl.f16, **shapes), ((100, k), (136, k))), (matmul_tn.trace(cl.bf16, **shapes), ((k, 104), (k, 136)))):
        if prog.name == "matmul_tn":
            prog = matmul_tn.trace(cl.bf16, M=104, N=136, K=k)
        ins = [((torch.rand(*shp, generator=g) * 2 - 1) / k ** 0.5).to(torch.bfloat16 if prog.name == "matmul_tn" else torch.float16)
               for shp in dims]
        want = po.evaluate(prog, ins)[0]
        print(f"case {prog.name} ragged K={k}", flush=True)
        got = kernel_for(prog, template="gemm", tiling=dict(BM=64, BN=64, BK=64, WM=2, WN=2))(*[t.cuda() for t in ins])
        np.testing.assert_allclose(got.float().cpu().numpy().reshape(want.shape), want, rtol=RTOL, atol=ATOL)
    bshapes = dict(BX=4, BW=2, M=70, N=64, K=k)
    _check(C.batched_matmul.trace(cl.f16, **bshapes), C.inputs_batched, bshapes)
    nshapes = dict(M=130, N=72, K=k)
    _check(C.rmsnorm_matmul.trace(cl.f16, **nshapes), C.inputs_c2, nshapes)
    _check(C.rmsnorm_matmul_eps.trace(cl.f16, **nshapes), C.inputs_plain_norm, nshapes)
