"""Kernel timing with HIP events, dispatch kept out of the timed region.

The reference captures ``batch`` launches in a CUDA graph and replays it so Python dispatch
does not pollute the reading (``python/cleave/runtime/timer.py:14-108``).  Here both the
capture and the replays happen inside the native library (``chip_time_graph``: ``batch``
launches per HIP graph, kernel nodes only, replayed between two events), and a plain launch
loop between two events on the launch stream (``chip_time_launches``) is kept beside it for
callers that want eager launches; kernels that are not ``CompiledKernel`` objects fall back
to a Python launch loop with a warning.
"""

from __future__ import annotations

import warnings


def time_rounds(body, repeats: int = 1) -> list:
    """Event milliseconds of ``body()`` for each of ``repeats`` rounds (torch's current stream)."""
    import torch

    rounds = []
    for _ in range(repeats):
        start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        body()
        stop.record()
        torch.cuda.synchronize()
        rounds.append(start.elapsed_time(stop))
    return rounds


def launch_rounds(kernel, args, launches: int, *, repeats: int = 1) -> list:
    """Milliseconds per round of ``launches`` plain calls (includes host dispatch)."""
    def body():
        for _ in range(launches):
            kernel(*args)

    return time_rounds(body, repeats)


def native_rounds(kernel, args, launches: int, *, repeats: int = 1, warmup: int = 0, rotate=None,
                  graph_batch: int = 0):
    """Milliseconds per round of ``launches`` launches issued by the native library (replays of
    a ``graph_batch``-launch HIP graph when that is > 0, else an eager loop), or None when
    ``kernel`` has no native timer."""
    timer = getattr(kernel, "time", None)
    if timer is None:
        return None
    rounds = []
    for i in range(repeats):
        rounds.append(timer(*args, warmup=warmup if i == 0 else 0, iters=launches, rotate=rotate,
                            graph_batch=min(graph_batch, launches)) * launches)
    return rounds


def mean_launch_ms(kernel, args, *, warmup: int = 0, iters: int = 1, batch: int = 100, rotate=None) -> float:
    """Mean ms per launch over at least ``iters`` launches, replayed ``batch`` to a graph."""
    if warmup < 0:
        raise ValueError(f"warmup_iters must be >= 0, got {warmup}")
    if iters <= 0:
        raise ValueError(f"profile_iters must be > 0, got {iters}")
    args = list(args)
    rounds = native_rounds(kernel, args, iters, warmup=warmup, rotate=rotate, graph_batch=batch)
    if rounds is not None:
        return rounds[0] / iters
    warnings.warn("kernel has no native timer; timing a Python launch loop, which includes per-call "
                  "dispatch overhead", RuntimeWarning, stacklevel=3)
    import torch

    for _ in range(warmup):
        kernel(*args)
    torch.cuda.synchronize()
    (elapsed,) = launch_rounds(kernel, args, iters)
    return elapsed / iters
