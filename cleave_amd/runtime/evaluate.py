"""Run tiling candidates through the workers and collect one typed result each.

Counterpart of ``python/cleave/runtime/evaluate.py:40-450``: codegen in the parent, compile +
validate (+ time) in up to ``max_parallel`` persistent workers, failures classified by stage
(``codegen`` / ``compile`` / ``validate`` / ``bench`` / ``timeout`` / ``crash``), per-candidate
timeouts that only cost the offending worker, an opt-in heartbeat.  The injectable stages
(``build_fn``, ``check_fn``, ``reference_fn``, ``pool``) keep their signatures.

hiprtc compiles are quick (well under a second per kernel), so the pool is mostly there to
contain faults; ``max_parallel=0`` runs every candidate in this process instead.
"""

from __future__ import annotations

import functools
import os
import shutil
import tempfile
import time
import traceback
from dataclasses import dataclass, replace
from multiprocessing.connection import wait as _wait_ready

from ..core.errors import (BenchmarkError, CandidateTimeout, CleaveError, CodegenError, CompileError, LdsExceeded,
                           ValidationError, WorkerCrash)
from ..core.settings import Settings
from .compile import CompilerPassOptions, _compile, _load_main_kernel_from_code, build_candidate_code, check_code
from .gpu import _create_parallel_env, _gpu_exec_guard
from .reference import graph_out_indices, make_inputs, order_inputs_for_kernel, placeholder_order
from .validate import BenchOptions, Tolerance, benchmark_compiled_kernel, publish_reference
from .workers import WorkerPool, _run_task


@dataclass
class CandidateResult:
    cand: object
    status: str                    # "ok" | "failed"
    stage: str | None = None       # codegen|compile|validate|bench|timeout|crash on failure
    error: CleaveError | None = None
    code: str | None = None
    cuda_src: str | None = None    # the device source the kernel was compiled from (HIP here)
    latency_ms: float | None = None
    label: str = ""

    @property
    def ok(self) -> bool:
        return self.status == "ok"

    @property
    def device_src(self):
        return self.cuda_src


# What the native library reports when a kernel asks for more LDS than a workgroup may own.
_LDS_MARKER = "LDS limit exceeded"
_TRACEBACK_LINES = 20


MAX_GPU_PROCESSES = 16     # processes that may hold the one GPU at once (parent included)


def _effective_compile_and_run_parallelism(max_parallel, io_bytes):
    """Cap workers so their inputs + outputs fit in 80 % of the free device memory, and so that
    workers plus this process stay within the number of processes one GPU is shared by."""
    max_parallel = min(max_parallel, MAX_GPU_PROCESSES - 1)
    try:
        import torch

        if not torch.cuda.is_available() or not io_bytes:
            return max_parallel
        free, _ = torch.cuda.mem_get_info()
        return max(1, min(max_parallel, int(free * 0.8) // io_bytes))
    except Exception:  # noqa: BLE001
        return max_parallel


def _candidate_progress_label(i, total, cand):
    return f"candidate {i}/{total} (rstep={cand.rstep_map}, output_tile={cand.output_tile})"


def _short_traceback(text):
    lines = text.strip().splitlines()
    if len(lines) > _TRACEBACK_LINES:
        lines = ["..."] + lines[-_TRACEBACK_LINES:]
    return "\n".join(lines)


def _restore_compile_error(result, label):
    """``(stage, typed error)`` for a worker's failure dict."""
    kind = result.get("error_type", "RuntimeError")
    message = result.get("error_message", "")
    trace = _short_traceback(result.get("traceback", ""))
    text = "\n".join(p for p in (f"{label} failed with {kind}", message, trace) if p)
    stage = result.get("stage") or "compile"
    if _LDS_MARKER in message or _LDS_MARKER in trace:
        return "compile", LdsExceeded(text)
    cls = {"validate": ValidationError, "bench": BenchmarkError}.get(stage, CompileError)
    return stage, cls(text)


def _parent_error(cls, label, what, exc):
    trace = _short_traceback("".join(traceback.format_exception(type(exc), exc, exc.__traceback__)))
    err = cls(f"{label} {what} failed with {type(exc).__name__}\n{exc}\n{trace}")
    err.__cause__ = exc
    return err


def _slowest(active, now, limit=3):
    jobs = sorted(active.values(), key=lambda j: now - j["started_at"], reverse=True)[:limit]
    return "; ".join(f"{j['label']} running {now - j['started_at']:.1f}s" for j in jobs)


def run_candidates(candidates, dtype, *, max_parallel: int = 8, tolerance: Tolerance | None = None,
                   timeout_s: float | None = None, compiler_pass_options: CompilerPassOptions | None = None,
                   benchmark: BenchOptions | None = None, build_fn=None, check_fn=None, reference_fn=None,
                   pool: WorkerPool | None = None) -> list:
    """Codegen, compile and validate every candidate; one ``CandidateResult`` each, in input order."""
    if not candidates:
        return []
    if build_fn is None:
        build_fn = functools.partial(build_candidate_code, options=compiler_pass_options or CompilerPassOptions())
    check_fn = check_fn or check_code
    reference_fn = reference_fn or publish_reference

    _create_parallel_env()
    settings = Settings.from_env()
    limit = settings.compile_timeout_secs if timeout_s is None else (timeout_s if timeout_s > 0 else None)
    log_on = settings.progress_log
    beat = settings.heartbeat_secs if log_on else None
    total = len(candidates)

    def fmt(v):
        return "disabled" if v is None else f"{v:g}s"

    if log_on:
        print(f"Compiling and running {total} scheduled graphs (max_parallel={max_parallel}, "
              f"timeout={fmt(limit)}, heartbeat={fmt(beat)}):", flush=True)
    else:
        print(f"Compiling and running {total} scheduled graphs:", flush=True)

    results = [None] * total
    runtime_root = settings.runtime_root
    os.makedirs(runtime_root, exist_ok=True)
    ref_root = tempfile.mkdtemp(prefix="ref_", dir=str(runtime_root))
    refs = {}  # id(flat_graph) -> (cache_dir, out_idx, io_bytes)

    def reference_for(cand):
        graph = cand.flat_graph
        if id(graph) not in refs:
            d = os.path.join(ref_root, f"g{len(refs)}")
            os.makedirs(d, exist_ok=True)
            out_idx, io_bytes = reference_fn(d, graph, dtype)
            refs[id(graph)] = (d, out_idx, io_bytes)
        return refs[id(graph)]

    def prepare(i, cand):
        """-> (job, task | None); a None task means the job already failed."""
        label = _candidate_progress_label(i, total, cand)
        job = {"idx": i, "candidate": cand, "label": label}
        try:
            ref_dir, out_idx, _ = reference_for(cand)
        except Exception as exc:  # noqa: BLE001
            results[i - 1] = CandidateResult(cand, "failed", "codegen", _parent_error(CleaveError, label, "reference", exc),
                                             label=label)
            return job, None
        try:
            code = build_fn(cand)
        except Exception as exc:  # noqa: BLE001
            results[i - 1] = CandidateResult(cand, "failed", "codegen", _parent_error(CodegenError, label, "codegen", exc),
                                             label=label)
            return job, None
        job["code_str"] = code
        return job, {"check_fn": check_fn, "code_str": code, "out_idx": out_idx, "reference_cache_dir": ref_dir,
                     "tolerance": tolerance, "benchmark": benchmark}

    def settle(job, result):
        cand, label, code = job["candidate"], job["label"], job.get("code_str")
        if result["ok"]:
            results[job["idx"] - 1] = CandidateResult(cand, "ok", None, None, code, result["cuda_src"],
                                                      result.get("latency_ms"), label)
        else:
            stage, err = _restore_compile_error(result, label)
            results[job["idx"] - 1] = CandidateResult(cand, "failed", stage, err, code=code, label=label)

    from tqdm import tqdm

    if max_parallel == 0:  # in-process: no isolation, no timeouts
        try:
            with tqdm(total=total, disable=None) as bar:
                for i, cand in enumerate(candidates, start=1):
                    job, task = prepare(i, cand)
                    if task is not None:
                        settle(job, _run_task(task))
                    bar.update(1)
        finally:
            shutil.rmtree(ref_root, ignore_errors=True)
        return results

    owns_pool = pool is None
    if owns_pool:
        pool = WorkerPool()
    active = {}
    todo = iter(enumerate(candidates, start=1))

    def fill(bar):
        while len(active) < max_parallel:
            try:
                i, cand = next(todo)
            except StopIteration:
                return
            job, task = prepare(i, cand)
            if task is None:
                bar.update(1)
                continue
            worker = None
            try:
                worker = pool.acquire()
                worker.conn.send(task)
            except Exception as exc:  # noqa: BLE001
                if worker is not None:
                    pool.discard(worker)
                results[i - 1] = CandidateResult(cand, "failed", "crash",
                                                 _parent_error(WorkerCrash, job["label"], "worker start", exc),
                                                 code=job["code_str"], label=job["label"])
                bar.update(1)
                continue
            job["started_at"] = time.monotonic()
            active[worker] = job

    def collect(bar):
        # a result is read before a death is noticed, so a worker that answered and then
        # retired is never counted as a crash
        for worker, job in list(active.items()):
            result, dead = worker.poll()
            if result is None and not dead:
                continue
            del active[worker]
            if result is not None:
                (pool.discard if result.get("retire") else pool.release)(worker)
                settle(job, result)
            else:
                worker.process.join(timeout=1.0)
                err = WorkerCrash(f"{job['label']} exited with code {worker.process.exitcode} before returning a result.")
                pool.discard(worker)
                results[job["idx"] - 1] = CandidateResult(job["candidate"], "failed", "crash", err,
                                                          code=job["code_str"], label=job["label"])
            bar.update(1)

    try:
        _, _, io_bytes = reference_for(candidates[0])
        max_parallel = _effective_compile_and_run_parallelism(max_parallel, io_bytes)
    except Exception:  # noqa: BLE001 - surfaces per candidate in prepare()
        pass
    try:
        with tqdm(total=total, disable=None) as bar:
            fill(bar)
            last_beat = time.monotonic()
            while active:
                now = time.monotonic()
                wait_s = 1.0
                if beat is not None:
                    wait_s = min(wait_s, max(0.0, beat - (now - last_beat)))
                if limit is not None:
                    oldest = min(j["started_at"] for j in active.values())
                    wait_s = min(wait_s, max(0.0, oldest + limit - now))
                _wait_ready([w.conn for w in active] + [w.process.sentinel for w in active], timeout=wait_s)
                collect(bar)
                now = time.monotonic()
                if limit is not None:
                    for worker, job in list(active.items()):
                        elapsed = now - job["started_at"]
                        if elapsed < limit:
                            continue
                        del active[worker]
                        pool.discard(worker)
                        err = CandidateTimeout(f"{job['label']} exceeded {limit:g}s after {elapsed:.1f}s; terminated worker.")
                        results[job["idx"] - 1] = CandidateResult(job["candidate"], "failed", "timeout", err,
                                                                  code=job["code_str"], label=job["label"])
                        bar.update(1)
                        if log_on:
                            print(f"[cleave] timed out {job['label']} after {elapsed:.1f}s", flush=True)
                if log_on and beat is not None and active and time.monotonic() - last_beat >= beat:
                    now = time.monotonic()
                    print(f"[cleave] {bar.n}/{total} done, {len(active)} running. Slowest: {_slowest(active, now)}",
                          flush=True)
                    last_beat = now
                fill(bar)
    finally:
        for worker in list(active):
            pool.discard(worker)
        if owns_pool:
            pool.close()
        shutil.rmtree(ref_root, ignore_errors=True)
    return results


class _SerialBench:
    """Recompile and time kernels one at a time in this process (after the workers)."""

    def __init__(self, dtype, warmup, iters):
        self.dtype, self.warmup, self.iters = dtype, warmup, iters
        self._inputs = {}

    def _inputs_for(self, graph):
        if id(graph) not in self._inputs:
            by_name = {ph.name: t for ph, t in zip(placeholder_order(graph), make_inputs(graph, self.dtype))}
            self._inputs[id(graph)] = (by_name, graph_out_indices(graph))
        return self._inputs[id(graph)]

    def latency_ms(self, graph, code_str):
        by_name, out_idx = self._inputs_for(graph)
        kernel = _compile(_load_main_kernel_from_code(code_str), out_idx)
        return benchmark_compiled_kernel(kernel, order_inputs_for_kernel(by_name, kernel),
                                         warmup_iters=self.warmup, profile_iters=self.iters)

    def close(self):
        self._inputs.clear()


def benchmark_results(results, dtype, warmup=16, iters=1000) -> list:
    """Copies of ``results`` with ``latency_ms`` re-measured serially on the ok ones; a kernel
    that fails to time comes back failed at stage ``bench``."""
    bench = _SerialBench(dtype, warmup, iters)
    timed = []
    try:
        for r in results:
            if not r.ok:
                timed.append(r)
                continue
            try:
                with _gpu_exec_guard():
                    latency = bench.latency_ms(r.cand.flat_graph, r.code)
            except Exception as exc:  # noqa: BLE001
                timed.append(replace(r, status="failed", stage="bench",
                                     error=_parent_error(BenchmarkError, r.label, "benchmark", exc)))
            else:
                timed.append(replace(r, latency_ms=latency))
    finally:
        bench.close()
    return timed
