"""The candidate runner and its worker pool with scripted stand-ins for the compile / validate / time
stages: no GPU and no compiler anywhere in the checked path.

A candidate here is a little script: ``{"sleep": s, "exit": code, "raise": kind, "stage": name}``.
The stand-in check function plays it inside the child and reports the child's pid as its
"latency", which is how the tests see which process did the work.
"""

import multiprocessing
import os
import time
from types import SimpleNamespace

import pytest

from cleave_amd.core import errors
from cleave_amd.runtime import workers
from cleave_amd.runtime.evaluate import STAGES, run_candidates

pytestmark = pytest.mark.skipif("fork" not in multiprocessing.get_all_start_methods(),
                                reason="the scripted stages live in this module: children must be forked")


def scripted(**script):
    return SimpleNamespace(script=script, rstep_map={"k": 32}, output_tile=[16, 16], flat_graph=None)


def emit(cand):
    if cand.script.get("codegen") == "refuse":
        raise KeyError("no template for this plan")
    return repr(sorted(cand.script.items()))


def play(code, *, out_idx, reference_cache_dir, tolerance=None, benchmark=None):
    script = dict(eval(code))      # the "source" is the script's repr
    time.sleep(script.get("sleep", 0.02))
    if "exit" in script:
        os._exit(script["exit"])
    if script.get("raise") == "mismatch":
        raise AssertionError("12 of 64 elements differ")
    if script.get("raise") == "staged":
        problem = RuntimeError("event timing failed")
        problem._cleave_stage = script["stage"]
        raise problem
    if script.get("raise") == "lds":
        raise RuntimeError("chip_launch: LDS limit exceeded: kernel asks for 200000 bytes, device allows 163840")
    if script.get("raise"):
        raise OSError("hiprtc: 3 errors generated")
    return f"compiled<{code}>", float(os.getpid())


def published(cache_dir, graph, dtype):
    assert os.path.isdir(cache_dir)
    return [-1], 0


def go(cands, pool=None, **kw):
    return run_candidates(cands, "float16", build_fn=emit, check_fn=play, reference_fn=published, pool=pool, **kw)


@pytest.fixture
def fork_pool():
    with workers.WorkerPool(multiprocessing.get_context("fork")) as pool:
        yield pool


def test_every_failure_kind_lands_on_its_own_candidate(fork_pool):
    cands = [scripted(), scripted(exit=7), scripted(**{"raise": "mismatch"}), scripted(**{"raise": "compiler"}),
             scripted(sleep=5.0), scripted(**{"raise": "staged", "stage": "bench"}), scripted(codegen="refuse"),
             scripted(**{"raise": "lds"}), scripted()]
    results = go(cands, fork_pool, max_parallel=3, timeout_s=0.6)
    assert [r.cand for r in results] == cands, "results come back in input order"
    assert [r.stage for r in results] == [None, "crash", "validate", "compile", "timeout", "bench", "codegen",
                                          "compile", None]
    assert all(r.stage in STAGES for r in results if not r.ok)
    kinds = [type(r.error) for r in results]
    assert kinds[1] is errors.WorkerCrash and "code 7" in str(results[1].error)
    assert kinds[2] is errors.ValidationError and isinstance(results[2].error, AssertionError)
    assert kinds[3] is errors.CompileError and "3 errors generated" in str(results[3].error)
    assert kinds[4] is errors.CandidateTimeout and isinstance(results[4].error, TimeoutError)
    assert kinds[5] is errors.BenchmarkError
    assert kinds[6] is errors.CodegenError and results[6].code is None and "no template" in str(results[6].error)
    assert kinds[7] is errors.LdsExceeded and errors.SmemExceeded is errors.LdsExceeded
    assert results[0].cuda_src.startswith("compiled<") and results[0].device_src == results[0].cuda_src
    assert results[4].code is not None, "a timed-out candidate keeps its generated source"


def test_children_are_kept_and_only_the_guilty_one_is_replaced(fork_pool):
    first = go([scripted(sleep=0.05) for _ in range(8)], fork_pool, max_parallel=2)
    pids = {r.latency_ms for r in first}
    assert len(pids) <= 2 and float(os.getpid()) not in pids
    assert set(map(float, fork_pool.pids)) == pids
    again = go([scripted(), scripted(exit=1), scripted()], fork_pool, max_parallel=1)
    assert again[0].latency_ms in pids, "a later call reuses the pool's children"
    assert again[2].ok and again[2].latency_ms != again[0].latency_ms, "the child that died was replaced"
    assert len(fork_pool.pids) <= 2


def test_time_limit_from_the_environment_and_heartbeat_lines(monkeypatch, capsys, fork_pool):
    monkeypatch.setenv("COMPILATION_PROGRESS_LOG", "1")
    monkeypatch.setenv("CLEAVE_COMPILE_AND_RUN_TIMEOUT_SECS", "0.4")
    monkeypatch.setenv("CLEAVE_COMPILE_PROGRESS_HEARTBEAT_SECS", "0.1")
    results = go([scripted(sleep=3.0), scripted(sleep=0.2)], fork_pool, max_parallel=2)
    assert [r.stage for r in results] == ["timeout", None]
    assert "exceeded 0.4s" in str(results[0].error)
    said = capsys.readouterr().out
    assert "max_parallel=2, timeout=0.4s, heartbeat=0.1s" in said
    assert "running. Slowest: candidate 1/2" in said and "[cleave] timed out candidate 1/2" in said


def test_quiet_unless_asked(monkeypatch, capsys, fork_pool):
    monkeypatch.delenv("COMPILATION_PROGRESS_LOG", raising=False)
    assert all(r.ok for r in go([scripted(), scripted()], fork_pool, max_parallel=2))
    assert capsys.readouterr().out.strip().splitlines() == ["Compiling and running 2 scheduled graphs:"]


def test_without_children_everything_runs_here():
    results = go([scripted(), scripted(**{"raise": "mismatch"})], max_parallel=0)
    assert results[0].ok and results[0].latency_ms == float(os.getpid())
    assert results[1].stage == "validate"
    assert go([], max_parallel=0) == []


def test_reference_is_published_once_per_graph(fork_pool):
    seen = []

    def counting(cache_dir, graph, dtype):
        seen.append((cache_dir, graph))
        return [-1], 0

    g1, g2 = object(), object()
    cands = [scripted(), scripted(), scripted()]
    cands[0].flat_graph = cands[2].flat_graph = g1
    cands[1].flat_graph = g2
    results = run_candidates(cands, "float16", build_fn=emit, check_fn=play, reference_fn=counting, pool=fork_pool,
                             max_parallel=2)
    assert all(r.ok for r in results)
    assert [g for _, g in seen] == [g1, g2] and len({d for d, _ in seen}) == 2
    assert not any(os.path.exists(d) for d, _ in seen), "the scratch directory is removed afterwards"


def test_pool_primitives(fork_pool):
    """submit / wait / abandon without the runner on top."""
    kwargs = {"out_idx": [-1], "reference_cache_dir": os.getcwd()}
    quick = fork_pool.submit({"check_fn": play, "code": emit(scripted()), "kwargs": kwargs}, tag="quick")
    stuck = fork_pool.submit({"check_fn": play, "code": emit(scripted(sleep=30.0)), "kwargs": kwargs}, tag="stuck")
    ended = []
    deadline = time.monotonic() + 5.0
    while not ended and time.monotonic() < deadline:
        ended = fork_pool.wait(0.2)
    assert [(t.tag, o.answer["ok"]) for t, o in ended] == [("quick", True)]
    assert [t.tag for t in fork_pool.tickets] == ["stuck"]
    victim = fork_pool._working[stuck].process.pid
    fork_pool.abandon(stuck)
    with pytest.raises(ProcessLookupError):
        os.kill(victim, 0)
    assert fork_pool.tickets == [] and fork_pool.wait(0.01) == []
    fork_pool.close()
    with pytest.raises(RuntimeError):
        fork_pool.submit({}, tag=None)


def test_execute_task_describes_failures_as_data():
    kwargs = {"out_idx": [-1], "reference_cache_dir": "."}
    good = workers.execute_task({"check_fn": play, "code": emit(scripted()), "kwargs": kwargs})
    assert good["ok"] and good["latency_ms"] == float(os.getpid())
    bad = workers.execute_task({"check_fn": play, "code": emit(scripted(**{"raise": "mismatch"})), "kwargs": kwargs})
    assert (bad["ok"], bad["stage"], bad["kind"]) == (False, "validate", "AssertionError") and "Traceback" in bad["trace"]
