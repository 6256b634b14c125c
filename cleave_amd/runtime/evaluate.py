"""Take a list of tiling candidates to one typed result each.

Service contract (the reference's ``python/cleave/runtime/evaluate.py:136-376`` gives its pipeline
the same one): source is generated in this process (``build_fn``), every candidate is then
checked -- compiled, validated against the published reference, timed -- by ``check_fn`` in a
child process of a ``WorkerPool``, at most ``max_parallel`` at once.  Whatever goes wrong is
attached to its candidate with the stage it happened in: ``codegen``, ``compile``, ``validate``,
``bench``, ``timeout`` (the child overstayed and was killed) or ``crash`` (the child died).  The
four injection points ``build_fn`` / ``check_fn`` / ``reference_fn`` / ``pool`` keep the
reference's signatures, so fakes written against it work here.

hiprtc compiles take a fraction of a second, so children are here to contain faults rather than
to gain speed; ``max_parallel=0`` checks everything in this process (no isolation, no time limit).
"""

from __future__ import annotations

import dataclasses
import os
import shutil
import tempfile
import time
import traceback
from collections import deque

from ..core import errors
from ..core.settings import Settings
from . import workers
from .compile import CompilerPassOptions, _compile, _load_main_kernel_from_code, build_candidate_code, check_code
from .gpu import _create_parallel_env, _gpu_exec_guard
from .reference import graph_out_indices, make_inputs, order_inputs_for_kernel, placeholder_order
from .validate import BenchOptions, Tolerance, benchmark_compiled_kernel, publish_reference
from .workers import WorkerPool

STAGES = ("codegen", "compile", "validate", "bench", "timeout", "crash")
GPU_PROCESS_LIMIT = 16          # processes that may share the one GPU, this one included
LDS_MARKER = "LDS limit exceeded"   # what the native library says when a kernel wants more LDS than a workgroup may own
KEPT_TRACE_LINES = 20


@dataclasses.dataclass
class CandidateResult:
    cand: object
    status: str                          # "ok" or "failed"
    stage: str | None = None             # one of STAGES when failed
    error: errors.CleaveError | None = None
    code: str | None = None              # generated source (None when codegen failed)
    cuda_src: str | None = None          # device source as compiled (HIP here; the field keeps the reference's name)
    latency_ms: float | None = None
    label: str = ""

    @property
    def ok(self) -> bool:
        return self.status == "ok"

    @property
    def device_src(self):
        return self.cuda_src


def _tail(text: str) -> str:
    rows = (text or "").strip().splitlines()
    return "\n".join(rows if len(rows) <= KEPT_TRACE_LINES else ["..."] + rows[-KEPT_TRACE_LINES:])


def _wrap(kind, label, activity, problem):
    """A typed error for something that failed in this process."""
    trace = _tail("".join(traceback.format_exception(type(problem), problem, problem.__traceback__)))
    wrapped = kind(f"{label} {activity} failed with {type(problem).__name__}\n{problem}\n{trace}")
    wrapped.__cause__ = problem
    return wrapped


def _typed_failure(answer: dict, label: str):
    """``(stage, error)`` from a child's failure dict."""
    body = "\n".join(part for part in (f"{label} failed with {answer.get('kind', 'RuntimeError')}",
                                       answer.get("text", ""), _tail(answer.get("trace", ""))) if part)
    if LDS_MARKER in body:
        return "compile", errors.LdsExceeded(body)
    stage = answer.get("stage") or "compile"
    if stage == "validate":
        return stage, errors.ValidationError(body)
    if stage == "bench":
        return stage, errors.BenchmarkError(body)
    return stage, errors.CompileError(body)


def _width_that_fits(requested: int, io_bytes: int) -> int:
    """Children to run at once: no more than share the GPU with this process, and no more than
    fit their inputs and outputs into four fifths of the free device memory."""
    width = min(requested, GPU_PROCESS_LIMIT - 1)
    if not io_bytes:
        return width
    try:
        import torch

        if torch.cuda.is_available():
            free = torch.cuda.mem_get_info()[0]
            width = max(1, min(width, (free * 4 // 5) // io_bytes))
    except Exception:  # noqa: BLE001 - without the figure the request stands
        pass
    return width


class _References:
    """Reference outputs, published once per flat graph under a scratch directory."""

    def __init__(self, publish, dtype, root):
        self.publish, self.dtype = publish, dtype
        self.root = tempfile.mkdtemp(prefix="ref_", dir=str(root))
        self.known = {}

    def of(self, cand):
        key = id(cand.flat_graph)
        if key not in self.known:
            where = os.path.join(self.root, f"g{len(self.known)}")
            os.makedirs(where, exist_ok=True)
            out_idx, io_bytes = self.publish(where, cand.flat_graph, self.dtype)
            self.known[key] = (where, out_idx, io_bytes)
        return self.known[key]

    def discard(self):
        shutil.rmtree(self.root, ignore_errors=True)


@dataclasses.dataclass
class _Job:
    slot: int                 # position in the input list
    cand: object
    label: str
    code: str | None = None
    task: dict | None = None
    began: float = 0.0

    def failed(self, stage, error):
        return CandidateResult(self.cand, "failed", stage, error, code=self.code, label=self.label)


class _Progress:
    """The bar, and the optional heartbeat lines."""

    def __init__(self, total, settings, limit, width):
        from tqdm import tqdm

        self.total, self.done = total, 0
        self.verbose = settings.progress_log
        self.every = settings.heartbeat_secs if self.verbose else None
        self.last = time.monotonic()
        head = f"Compiling and running {total} scheduled graphs"
        if self.verbose:
            show = lambda v: "disabled" if v is None else f"{v:g}s"    # noqa: E731
            head += f" (max_parallel={width}, timeout={show(limit)}, heartbeat={show(self.every)})"
        print(head + ":", flush=True)
        self.bar = tqdm(total=total, disable=None)

    def tick(self):
        self.done += 1
        self.bar.update(1)

    def say(self, text):
        if self.verbose:
            print(f"[cleave] {text}", flush=True)

    def until_beat(self, now):
        return None if self.every is None else max(0.0, self.every - (now - self.last))

    def beat(self, running, now):
        if self.every is None or not running or now - self.last < self.every:
            return
        oldest = sorted(running, key=lambda job: job.began)[:3]
        self.say(f"{self.done}/{self.total} done, {len(running)} running. Slowest: "
                 + "; ".join(f"{job.label} running {now - job.began:.1f}s" for job in oldest))
        self.last = now

    def close(self):
        self.bar.close()


def run_candidates(candidates, dtype, *, max_parallel: int = 8, tolerance: Tolerance | None = None,
                   timeout_s: float | None = None, compiler_pass_options: CompilerPassOptions | None = None,
                   benchmark: BenchOptions | None = None, build_fn=None, check_fn=None, reference_fn=None,
                   pool: WorkerPool | None = None) -> list:
    """One ``CandidateResult`` per candidate, in input order.

    ``timeout_s``: seconds a child may spend on one candidate (None: the environment's setting,
    <= 0: no limit).  ``pool``: children to reuse (left open); otherwise a pool is made and closed."""
    candidates = list(candidates)
    if not candidates:
        return []
    if build_fn is None:
        options = compiler_pass_options or CompilerPassOptions()
        build_fn = lambda cand: build_candidate_code(cand, options=options)    # noqa: E731
    check_fn = check_fn or check_code
    _create_parallel_env()
    settings = Settings.from_env()
    if timeout_s is None:
        limit = settings.compile_timeout_secs
    else:
        limit = timeout_s if timeout_s > 0 else None
    os.makedirs(settings.runtime_root, exist_ok=True)
    references = _References(reference_fn or publish_reference, dtype, settings.runtime_root)
    results: list = [None] * len(candidates)
    progress = _Progress(len(candidates), settings, limit, max_parallel)

    def prepared(slot, cand):
        """The job with source and task filled in, or None after recording why it cannot run."""
        job = _Job(slot, cand, f"candidate {slot + 1}/{len(candidates)} (rstep={cand.rstep_map}, "
                               f"output_tile={cand.output_tile})")
        try:
            where, out_idx, _ = references.of(cand)
        except Exception as problem:  # noqa: BLE001
            results[slot] = job.failed("codegen", _wrap(errors.CleaveError, job.label, "reference", problem))
            return None
        try:
            job.code = build_fn(cand)
        except Exception as problem:  # noqa: BLE001
            results[slot] = job.failed("codegen", _wrap(errors.CodegenError, job.label, "codegen", problem))
            return None
        job.task = {"check_fn": check_fn, "code": job.code,
                    "kwargs": {"out_idx": out_idx, "reference_cache_dir": where, "tolerance": tolerance,
                               "benchmark": benchmark}}
        return job

    def record(job, answer):
        if answer["ok"]:
            results[job.slot] = CandidateResult(job.cand, "ok", code=job.code, cuda_src=answer["device_src"],
                                                latency_ms=answer.get("latency_ms"), label=job.label)
        else:
            results[job.slot] = job.failed(*_typed_failure(answer, job.label))

    try:
        if max_parallel == 0:
            for slot, cand in enumerate(candidates):
                job = prepared(slot, cand)
                if job is not None:
                    record(job, workers.execute_task(job.task))
                progress.tick()
            return results
        _in_children(candidates, prepared, record, results, progress, references, limit, max_parallel, pool)
        return results
    finally:
        progress.close()
        references.discard()


def _in_children(candidates, prepared, record, results, progress, references, limit, width, pool):
    """The scheduling loop: keep up to ``width`` children busy, collect answers and deaths, kill
    children that overstay ``limit`` seconds."""
    try:
        width = _width_that_fits(width, references.of(candidates[0])[2])
    except Exception:  # noqa: BLE001 - every candidate then records this failure itself
        pass
    own_pool = pool is None
    pool = pool or WorkerPool()
    waiting = deque(enumerate(candidates))
    running: dict = {}          # ticket -> job

    def start_more():
        while waiting and len(running) < width:
            job = prepared(*waiting.popleft())
            if job is None:
                progress.tick()
                continue
            try:
                ticket = pool.submit(job.task, tag=job.slot)
            except Exception as problem:  # noqa: BLE001
                results[job.slot] = job.failed("crash", _wrap(errors.WorkerCrash, job.label, "worker start", problem))
                progress.tick()
                continue
            job.began = time.monotonic()
            running[ticket] = job

    try:
        start_more()
        while running:
            now = time.monotonic()
            pause = 1.0
            if limit is not None:
                pause = min(pause, max(0.0, min(job.began for job in running.values()) + limit - now))
            beat_in = progress.until_beat(now)
            if beat_in is not None:
                pause = min(pause, beat_in)
            for ticket, outcome in pool.wait(pause):
                job = running.pop(ticket)
                if outcome.answer is not None:
                    record(job, outcome.answer)
                else:
                    results[job.slot] = job.failed("crash", errors.WorkerCrash(
                        f"{job.label} exited with code {outcome.exit_code} before returning a result."))
                progress.tick()
            now = time.monotonic()
            if limit is not None:
                for ticket, job in [(t, j) for t, j in running.items() if now - j.began >= limit]:
                    del running[ticket]
                    pool.abandon(ticket)
                    spent = now - job.began
                    results[job.slot] = job.failed("timeout", errors.CandidateTimeout(
                        f"{job.label} exceeded {limit:g}s after {spent:.1f}s; terminated worker."))
                    progress.tick()
                    progress.say(f"timed out {job.label} after {spent:.1f}s")
            progress.beat(list(running.values()), time.monotonic())
            start_more()
    finally:
        for ticket in list(running):
            pool.abandon(ticket)
        if own_pool:
            pool.close()


# --------------------------------------------------------------------------- serial re-timing
def benchmark_results(results, dtype, warmup=16, iters=1000) -> list:
    """The same results with ``latency_ms`` measured again, one kernel at a time in this process
    (after the children are gone, so nothing else is on the GPU).  A kernel that cannot be timed
    comes back failed at stage ``bench``; failed results pass through."""
    inputs_of = {}

    def inputs_for(graph):
        if id(graph) not in inputs_of:
            tensors = dict(zip((ph.name for ph in placeholder_order(graph)), make_inputs(graph, dtype)))
            inputs_of[id(graph)] = (tensors, graph_out_indices(graph))
        return inputs_of[id(graph)]

    timed = []
    for result in results:
        if not result.ok:
            timed.append(result)
            continue
        try:
            with _gpu_exec_guard():
                tensors, out_idx = inputs_for(result.cand.flat_graph)
                kernel = _compile(_load_main_kernel_from_code(result.code), out_idx)
                latency = benchmark_compiled_kernel(kernel, order_inputs_for_kernel(tensors, kernel),
                                                    warmup_iters=warmup, profile_iters=iters)
        except Exception as problem:  # noqa: BLE001
            timed.append(dataclasses.replace(result, status="failed", stage="bench",
                                             error=_wrap(errors.BenchmarkError, result.label, "benchmark", problem)))
        else:
            timed.append(dataclasses.replace(result, latency_ms=latency))
    return timed
