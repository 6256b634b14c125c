"""Frontend: tracing, record kinds, eager dispatch, fingerprints, refusals, paged recognition
(the scenarios of the reference's tests/frontend/test_program.py and test_exact_softmax.py)."""

import numpy as np
import pytest
import torch

import cleave_amd
import cleave_amd.lang as cl
from cleave_amd.core.errors import CleaveError, SpecError
from cleave_amd.frontend import Program, trace
from cleave_amd import examples as C


def softmax(x: cl.Tensor["R", "C"]):
    return cl.softmax(x, -1)


def softmax_shift(x: cl.Tensor["R", "C"]):
    return cl.softmax(x, -1, shift=-4.0)


def kinds(prog):
    return [r.kind for r in prog.ops]


def test_reference_matmul_and_named_binding():
    prog = C.matmul.trace(M=16, N=8, K=32)
    x, w = prog.random_inputs(device="cpu")
    (y,) = prog.reference(x, w)
    assert y.dtype == torch.float16 and y.shape == (16, 8)
    torch.testing.assert_close(y.float(), x.float() @ w.float(), rtol=2e-2, atol=2e-2)
    torch.testing.assert_close(prog.reference(w=w, x=x)[0], y)
    with pytest.raises(SpecError):
        prog.reference(torch.zeros(16, 31), torch.zeros(31, 8))
    with pytest.raises(TypeError):
        prog.reference(torch.zeros(16, 32))


def test_exact_softmax_traces_max_and_sub():
    prog = trace(softmax, {"R": 4, "C": 32}, cl.f32)
    assert kinds(prog) == ["input", "reduce_max", "sub", "exp", "reduce_sum", "div"]
    assert prog.ops[1].attr("dim") == 1 and prog.value(prog.ops[1].out).shape == (4, 1)
    ops = [o["op_type"] for o in prog.to_graph_structure()]
    assert ops == ["kn_input_op", "kn_reduce_max_1_op", "kn_sub_op", "kn_exp_op", "kn_reduce_sum_1_op", "kn_div_op",
                   "kn_output_op"]
    x = torch.randn(4, 32) * 30
    torch.testing.assert_close(prog.reference(x)[0], torch.softmax(x, -1))
    assert kinds(trace(softmax_shift, {"R": 4, "C": 32}, cl.f32)) == ["input", "add", "exp", "reduce_sum", "div"]


def test_builder_records_and_refusals():
    p = Program("p", cl.f32)
    a, b = p.input("a", [4, 8]), p.input("b", [4, 1])
    p.output(a - b), p.output(b - a), p.output(a.max(0, keepdim=True)), p.output(cl.max(a, -1, keepdim=True))
    assert [(r.kind, r.args) for r in p.ops[2:]] == [("sub", (0, 1)), ("sub", (1, 0)), ("reduce_max", (0,)),
                                                     ("reduce_max", (0,))]
    assert [r.attr("dim") for r in p.ops[4:]] == [0, 1]
    with pytest.raises(SpecError, match="keepdim"):
        a.max(-1)
    with pytest.raises(SpecError, match="out of range"):
        a.max(2, keepdim=True)
    with pytest.raises(SpecError, match="broadcastable"):
        a - p.input("c", [4, 3])
    with pytest.raises(SpecError, match="duplicate"):
        p.input("a", [4, 8])
    with pytest.raises(SpecError):
        bool(a)
    with pytest.raises(SpecError, match="transposed"):
        p.output(a.mT)
    assert (2.0 * a).id != a.id and p.ops[-1].args == (0, 2.0)       # scalar kept on the right


def test_eager_dispatch_and_jit_without_kernel():
    x = torch.randn(4, 8) * 20
    torch.testing.assert_close(cl.softmax(x, -1), torch.softmax(x, -1))
    torch.testing.assert_close(cl.max(x, 1, keepdim=True), x.amax(1, keepdim=True))
    f = cleave_amd.jit(softmax)
    torch.testing.assert_close(f.eager(x), torch.softmax(x, -1))
    with pytest.raises(CleaveError, match="compile"):
        f(x)                                                        # never a silent eager evaluation


def test_fingerprint_is_structural():
    a = C.gqa_decode_exact.trace(HQ=4, HKV=4, SQ=8, SKV=32, D=16).fingerprint()
    assert a == C.gqa_decode_exact.trace(HQ=4, HKV=4, SQ=8, SKV=32, D=16).fingerprint() and len(a) == 64
    assert a != C.gqa_decode_exact.trace(HQ=4, HKV=4, SQ=8, SKV=64, D=16).fingerprint()
    assert trace(C.matmul, dict(M=16, N=8, K=32), cl.bf16).fingerprint() != C.matmul.trace(M=16, N=8, K=32).fingerprint()


def test_trace_refusals():
    with pytest.raises(SpecError, match="not dims"):
        trace(C.matmul, dict(M=1, N=1, K=1, Z=3))
    with pytest.raises(SpecError, match="unbound"):
        trace(C.matmul, dict(M=1, N=1))
    prog = C.matmul.trace(M=4, N=4, K=8)
    assert prog.can_split("K") == [(False, True), (True, False)]
    with pytest.raises(SpecError, match="split dims"):
        prog.can_split("Q")


def test_random_inputs_are_positive_where_needed():
    p = Program("p", cl.f32)
    a, b = p.input("a", [4, 4]), p.input("b", [4, 4])
    p.output(a.sqrt() / b)
    x, y = p.random_inputs(seed=3, device="cpu")
    assert (x > 0).all() and (y > 0).all()
    x2, _ = p.random_inputs(seed=3, device="cpu")
    assert torch.equal(x, x2)


# ----------------------------------------------------------------------------- paged programs
batch, num_pages, n_idx = cl.dims("batch num_pages n_idx", dynamic=True)
kv_len = cl.Dim("kv_len", dynamic=True, hint=4096)


def paged_op(H_Q=32, H_KV=8, D=128, PAGE=1):
    @cleave_amd.jit(name=f"gqa_paged_decode_h{H_Q}_kv{H_KV}_d{D}_ps{PAGE}", dtype=cl.bf16)
    def op(q: cl.Tensor[batch, H_Q, D], k_cache: cl.Tensor[num_pages, PAGE, H_KV, D],
           v_cache: cl.Tensor[num_pages, PAGE, H_KV, D], kv_indptr: cl.Tensor[batch + 1, cl.i32],
           kv_indices: cl.Tensor[n_idx, cl.i32], kv_last_page_len: cl.Tensor[batch, cl.i32] | None,
           sm_scale: cl.Scalar[cl.f32]):
        pages = cl.PageTable(kv_indptr, kv_indices, last_page_len=kv_last_page_len, length=kv_len)
        k, v = cl.paged_gather(k_cache, pages), cl.paged_gather(v_cache, pages)
        qg = q.view(batch, H_KV, H_Q // H_KV, D)
        p, lse = cl.softmax((qg @ k.mT) * sm_scale, dim=-1, return_lse=True)
        return (p @ v).view(batch, H_Q, D), lse.view(batch, H_Q)

    return op


def test_paged_program_is_recognised():
    from cleave_amd.frontend.paged import is_paged, trace_paged

    op = paged_op(PAGE=64)
    assert is_paged(op) and not is_paged(C.matmul)
    att = trace_paged(op).attention()
    assert (att.num_qo_heads, att.num_kv_heads, att.head_dim, att.page_size) == (32, 8, 128, 64)
    assert not att.is_mla and not att.is_prefill and att.kind == "paged_decode_slab" and att.query_rows == 16
    spec = att.paging_spec()
    assert spec.last_page_len_input == "KV_LAST_PAGE_LEN" and spec.scale_input == "sm_scale" and spec.group == 4
    assert [p.name for p in att.inputs] == ["q", "k_cache", "v_cache", "kv_indptr", "kv_indices", "kv_last_page_len",
                                             "sm_scale"]
    body = att.dense_body()
    assert [s.name for s in body.inputs] == ["Q", "K", "V"] and body.inputs[1].shape == (4096, 128)
    # one token per page: the optional last_page_len is dropped from the kernel's inputs
    att1 = trace_paged(paged_op(PAGE=1)).attention()
    assert att1.kind == "paged_decode" and "kv_last_page_len" not in [p.name for p in att1.inputs]


def test_paged_program_refusals():
    from cleave_amd.frontend.paged import PagedProgram, trace_paged

    with pytest.raises(SpecError, match="dense program"):
        PagedProgram("p").apply("sub", (None, None))

    @cleave_amd.jit(dtype=cl.bf16)
    def unscaled(q: cl.Tensor[batch, 8, 64], kc: cl.Tensor[num_pages, 1, 2, 64], vc: cl.Tensor[num_pages, 1, 2, 64],
                 ptr: cl.Tensor[batch + 1, cl.i32], idx: cl.Tensor[n_idx, cl.i32], s: cl.Scalar[cl.f32]):
        pages = cl.PageTable(ptr, idx)
        k, v = cl.paged_gather(kc, pages), cl.paged_gather(vc, pages)
        return cl.softmax(q.view(batch, 2, 4, 64) @ k.mT, dim=-1) @ v

    with pytest.raises(SpecError, match=r"scores \* cl.Scalar"):
        trace_paged(unscaled).attention()
    with pytest.raises(SpecError, match="paged dims are dynamic"):
        trace(paged_op(), dict(batch=4))


def test_paged_decode_workloads_are_deterministic():
    wl = cl.workloads.paged_decode(batch=(1, 7), kv_len=(16, 1024), samples=3)
    assert wl.axes() == [(1, 16), (1, 128), (1, 1024), (7, 16), (7, 128), (7, 1024)]
    lens = wl.lengths(7, 1024)
    assert lens == wl.lengths(7, 1024) and lens[0] == 1024 and all(512 <= n <= 1024 for n in lens)


def test_paged_program_survives_its_plain_data_form():
    """A compiled paged operator is saved as JSON, not as a pickle: the program must come back
    from ``to_doc()`` recognisable as the same operator."""
    import json

    from cleave_amd.frontend.paged import PagedProgram, trace_paged

    op = paged_op(PAGE=64)
    program = trace_paged(op)
    program.split = (cl.Split("kv_len", (4, 8)),)
    back = PagedProgram.from_doc(json.loads(json.dumps(program.to_doc())))
    assert repr(back) == repr(program) and back.split == program.split
    a, b = program.attention(), back.attention()
    assert a.paging_spec() == b.paging_spec() and a.kind == b.kind
    assert [p.name for p in a.inputs] == [p.name for p in b.inputs]
    assert a.output_dims() == b.output_dims() and a.dense_body().fingerprint() == b.dense_body().fingerprint()
    with pytest.raises(SpecError, match="format"):
        PagedProgram.from_doc({"format": 7})


def test_settings_and_sessions(monkeypatch, tmp_path):
    from cleave_amd.core import Session, Settings, active_session, current_session

    env = {"CLEAVE_COMPILE_AND_RUN_TIMEOUT_SECS": "0", "CLEAVE_COMPILE_PROGRESS_HEARTBEAT_SECS": "junk",
           "COMPILATION_PROGRESS_LOG": " Yes ", "CLEAVE_TEST_SEED": str(2 ** 32 + 5), "SCRATCH": str(tmp_path)}
    s = Settings.from_env(env)
    assert s.compile_timeout_secs is None and s.heartbeat_secs == 15.0 and s.progress_log and s.test_seed == 5
    assert s.cache_root == tmp_path / "cleave_cache" and s.runtime_root == s.cache_root / "runtime"
    assert Settings.from_env({"CLEAVE_CACHE_ROOT": str(tmp_path / "x"), "SCRATCH": "/nowhere"}).cache_root == tmp_path / "x"
    assert s.replace(progress_log=False) != s and s.replace() == s
    with pytest.raises(AttributeError):
        s.progress_log = False
    assert active_session() is None
    with Session(cache_root=tmp_path / "a", max_parallel=3) as outer:
        with Session(settings=s) as inner:
            assert current_session() is inner and inner.cache_root == s.cache_root
            with pytest.raises(RuntimeError):
                outer.__exit__(None, None, None)
        assert active_session() is outer and outer.max_parallel == 3
    assert active_session() is None
    with pytest.raises(ValueError):
        Session(max_parallel=0)
