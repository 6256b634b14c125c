"""``run_candidates`` with injected fake stages on a fork pool: timeout, crash and validation
failures are classified, only the offending worker is replaced, workers are reused.  No GPU
and no compiler in the checked path (the scenarios of the reference's
``tests/test_runtime_parallel.py``)."""

import multiprocessing as mp
import os
import time
from types import SimpleNamespace

import pytest

from cleave_amd.core.errors import CandidateTimeout, ValidationError, WorkerCrash
from cleave_amd.runtime.evaluate import run_candidates
from cleave_amd.runtime.workers import WorkerPool

pytestmark = pytest.mark.skipif("fork" not in mp.get_all_start_methods(), reason="requires fork")


def _build(cand):
    return cand.code


def _no_reference(cache_dir, graph, dtype):
    return [-1], 0


def _check(code_str, *, out_idx, reference_cache_dir, tolerance=None, benchmark=None):
    """The code string says what the fake candidate does; the 'latency' is the worker's pid."""
    if code_str == "slow":
        time.sleep(1.0)
    elif code_str == "crash":
        os._exit(3)
    elif code_str == "wrong":
        raise AssertionError("mismatch")
    else:
        time.sleep(0.15 if code_str.startswith("fast") else 0.05)
    return f"hip_{code_str}", os.getpid()


def _cands(*codes):
    return [SimpleNamespace(code=c, rstep_map={"id": i}, output_tile=(i,), flat_graph=None)
            for i, c in enumerate(codes, start=1)]


@pytest.fixture
def pool():
    with WorkerPool(mp.get_context("fork")) as p:
        yield p


def _run(cands, pool, **kw):
    return run_candidates(cands, "float16", build_fn=_build, check_fn=_check, reference_fn=_no_reference, pool=pool, **kw)


def test_timeout_and_heartbeat(monkeypatch, capsys, pool):
    monkeypatch.setenv("COMPILATION_PROGRESS_LOG", "true")
    monkeypatch.setenv("CLEAVE_COMPILE_AND_RUN_TIMEOUT_SECS", "0.3")
    monkeypatch.setenv("CLEAVE_COMPILE_PROGRESS_HEARTBEAT_SECS", "0.05")
    results = _run(_cands("fast_a", "slow", "fast_b"), pool, max_parallel=2)
    assert [r.code for r in results if r.ok] == ["fast_a", "fast_b"]
    (bad,) = [r for r in results if not r.ok]
    assert bad.cand.code == "slow" and isinstance(bad.error, TimeoutError) and "candidate 2/3" in str(bad.error)
    out = capsys.readouterr().out
    assert "[cleave]" in out and "2 running. Slowest: candidate 2/3" in out
    assert "[cleave] timed out candidate 2/3" in out


def test_progress_log_is_off_by_default(monkeypatch, capsys, pool):
    monkeypatch.delenv("COMPILATION_PROGRESS_LOG", raising=False)
    monkeypatch.setenv("CLEAVE_COMPILE_PROGRESS_HEARTBEAT_SECS", "0.01")
    results = _run(_cands("fast_a", "fast_b"), pool, max_parallel=2)
    assert all(r.ok for r in results)
    assert capsys.readouterr().out == "Compiling and running 2 scheduled graphs:\n"


def test_workers_are_reused(pool):
    cands = _cands(*(f"c{i}" for i in range(6)))
    first = _run(cands, pool, max_parallel=2)
    assert [r.cuda_src for r in first] == [f"hip_c{i}" for i in range(6)]
    pids = {r.latency_ms for r in first}
    assert len(pids) <= 2 and os.getpid() not in pids
    second = _run(cands[:2], pool, max_parallel=2)
    assert {r.latency_ms for r in second} <= pids


def test_crash_timeout_and_wrong_answer_are_classified(pool):
    cands = _cands("a", "crash", "b", "slow", "wrong", "c")
    results = _run(cands, pool, max_parallel=1, timeout_s=0.5)
    assert [r.cand for r in results] == cands
    assert [r.stage for r in results] == [None, "crash", None, "timeout", "validate", None]
    assert isinstance(results[1].error, WorkerCrash) and "exited with code 3" in str(results[1].error)
    assert isinstance(results[3].error, CandidateTimeout)
    assert isinstance(results[4].error, ValidationError) and isinstance(results[4].error, AssertionError)
    a, b, c = results[0].latency_ms, results[2].latency_ms, results[5].latency_ms
    assert a != b != c   # a fresh worker after the crash and after the timeout
    assert len(pool.pids) == 1


def test_codegen_failure_stays_in_the_parent(pool):
    def build(cand):
        if cand.code == "nogen":
            raise ValueError("cannot emit")
        return cand.code

    results = run_candidates(_cands("a", "nogen"), "float16", build_fn=build, check_fn=_check,
                             reference_fn=_no_reference, pool=pool, max_parallel=2)
    assert results[0].ok and results[1].stage == "codegen" and "cannot emit" in str(results[1].error)


def test_in_process_mode_needs_no_pool():
    results = run_candidates(_cands("a", "wrong"), "float16", build_fn=_build, check_fn=_check,
                             reference_fn=_no_reference, max_parallel=0)
    assert results[0].ok and results[0].latency_ms == os.getpid()
    assert results[1].stage == "validate"
