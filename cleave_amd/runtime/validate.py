"""Tolerances, the on-disk reference a worker validates against, and the check itself
(``python/cleave/runtime/validate.py:19-197``)."""

from __future__ import annotations

import contextlib
import os
from dataclasses import dataclass
from pathlib import Path

from .gpu import _gpu_exec_guard
from .timer import mean_launch_ms


@dataclass(frozen=True)
class Tolerance:
    rtol: float
    atol: float
    equal_nan: bool = False


# The loose default bound of the reference; per-operator tolerances tighten it.
DEFAULT_TOLERANCE = Tolerance(rtol=0.5, atol=0.5)
# What every selected candidate of this back end is held to against the fp32-accumulated reference.
STRICT_TOLERANCE = Tolerance(rtol=1e-2, atol=1e-2)


@dataclass(frozen=True)
class BenchOptions:
    warmup: int = 16
    iters: int = 1000


@contextlib.contextmanager
def _stage(name):
    """Tag an escaping exception with the stage (compile / validate / bench) it came from."""
    try:
        yield
    except BaseException as exc:
        if getattr(exc, "_cleave_stage", None) is None:
            try:
                exc._cleave_stage = name
            except Exception:  # noqa: BLE001 - some builtins refuse attributes
                pass
        raise


def _live_bytes(tensors) -> int:
    return sum(t.element_size() * t.nelement() for t in tensors)


_BENCH_BATCH = 100


_LAST_LEVEL_CACHE = 256 << 20      # bytes of memory-side cache in front of HBM on this part


def rotation_sets(input_tensors) -> list | None:
    """Copies of the inputs to rotate through while timing, or None.  Inputs between 1/16 of and
    twice the memory-side cache (256 MB here) would be served from that cache, wholly or in part (a
    269 MB working set still finds a good share of itself there), by every launch after the first,
    and candidates would be ranked by a speed no caller sees (a decode step streams weights or a KV
    cache that other work has evicted since): enough copies are made that consecutive launches read
    different memory, at least twice the cache in total.  Smaller inputs stay cached in real use as
    well; larger ones stream anyway."""
    tensors = [t for t in input_tensors if hasattr(t, "element_size")]
    live = _live_bytes(tensors)
    if not (_LAST_LEVEL_CACHE // 16 <= live < 2 * _LAST_LEVEL_CACHE):
        return None
    copies = min(8, -(-2 * _LAST_LEVEL_CACHE // live)) - 1
    return [[t.clone() if hasattr(t, "element_size") else t for t in input_tensors] for _ in range(copies)]


def benchmark_compiled_kernel(kernel, input_tensors, *, warmup_iters=0, profile_iters=1) -> float:
    """Mean milliseconds per launch of ``kernel(*input_tensors)`` (over rotating copies of
    cache-sized inputs: see ``rotation_sets``)."""
    return mean_launch_ms(kernel, input_tensors, warmup=warmup_iters, iters=profile_iters, batch=_BENCH_BATCH,
                          rotate=rotation_sets(input_tensors))


class _ReferenceFile:
    """Inputs and expected outputs of one graph as a file the children read: written once by the
    parent (to a temporary name, then moved into place), loaded with ``weights_only`` so that
    nothing in it is executed.  It also records how the outputs are to be compared."""

    NAME = "reference.pt"

    def __init__(self, folder):
        self.folder = Path(folder)
        self.path = self.folder / self.NAME

    def write(self, inputs_by_name, reference, compare):
        import torch

        self.folder.mkdir(parents=True, exist_ok=True)
        scratch = self.path.with_name(f"{self.NAME}.tmp.{os.getpid()}")
        torch.save({"inputs_by_name": {name: t.cpu() for name, t in inputs_by_name.items()},
                    "reference": [t.cpu() for t in reference], "compare": compare}, scratch)
        os.replace(scratch, self.path)

    def read(self, device="cuda") -> tuple:
        """``(inputs by name, expected outputs, compare mode)``."""
        import torch

        held = torch.load(self.path, map_location=device, weights_only=True)
        return dict(held["inputs_by_name"]), list(held["reference"]), held.get("compare", "plain")


def _reference_path(cache_dir) -> Path:
    return _ReferenceFile(cache_dir).path


def compare_mode(graph) -> str:
    """How a stage's raw outputs are compared.  Softmax partials (m, l, O) are sums relative to a
    reference point m that a kernel is free to choose (the running maximum, a maximum raised
    only in coarse steps, or the log-sum-exp itself with l = 1 and normalised values), so they
    are compared as (m + log2 l, O / l): the quantities that do not depend on that choice and
    that the combine actually consumes."""
    low = getattr(graph, "lowered", None)
    if low is not None and getattr(graph, "role", "main") == "partial" and low.family in ("attention", "mla"):
        return "softmax_partial"
    return "plain"


def publish_reference(reference_cache_dir, graph, dtype, device: str = "cuda"):
    """The parent's side: inputs and reference of ``graph`` built once and left in
    ``reference_cache_dir`` for the children.  Returns ``(out_idx, io_bytes)``; ``io_bytes`` (what
    one child will hold on the device) sizes how many children may run at once."""
    import torch

    from .reference import build_inputs_and_reference

    with _gpu_exec_guard():
        inputs_by_name, reference, out_idx = build_inputs_and_reference(graph, dtype, device)
        io_bytes = _live_bytes(inputs_by_name.values()) + _live_bytes(reference)
        _ReferenceFile(reference_cache_dir).write(inputs_by_name, reference, compare_mode(graph))
        del inputs_by_name, reference
        if torch.cuda.is_available():
            torch.cuda.synchronize()
            torch.cuda.empty_cache()
    return out_idx, io_bytes


def _load_reference(reference_cache_dir, device: str = "cuda", with_mode: bool = False):
    inputs_by_name, reference, mode = _ReferenceFile(reference_cache_dir).read(device)
    return (inputs_by_name, reference, mode) if with_mode else (inputs_by_name, reference)


def _comparable(outputs, mode):
    if mode not in ("softmax_partial", "softmax_partial_folded"):
        return list(outputs)
    import torch

    pm, pl, po = (t.float() for t in outputs)
    if mode == "softmax_partial_folded":
        # a kernel that cuts the keys into ranges of its own (every key in exactly one of them): what
        # does not depend on the cut is the fold of all ranges, the quantity the combine makes of them
        m = pm.amax(0, keepdim=True)
        f = torch.exp2(pm - m)
        pm, pl, po = m[0], (pl * f).sum(0), (po * f.unsqueeze(-1)).sum(0)
    lse = torch.where(pl > 0, pm + torch.log2(pl.clamp_min(1e-30)), torch.full_like(pm, -1.0e30))
    return [lse, po / pl.clamp_min(1e-30).unsqueeze(-1)]


def own_cut(kernel) -> bool:
    """Whether a split kernel deals the keys out to its ranges by a rule of its own (the skewed
    ranges of the streaming decode kernel) rather than in equal shares."""
    tiling = getattr(kernel, "manifest", {}).get("tiling") or {}
    return bool(tiling.get("SKEW"))


def _validate_kernel_outputs(kernel, inputs, reference, *, tolerance: Tolerance = DEFAULT_TOLERANCE,
                             compare: str = "plain"):
    """Run ``kernel(*inputs)`` and assert every output is within ``tolerance`` of ``reference``."""
    import torch

    from .reference import reconcile_output_layout

    produced = kernel(*inputs)
    produced = list(produced) if isinstance(produced, (tuple, list)) else [produced]
    torch.cuda.synchronize()
    if len(produced) != len(reference):
        raise AssertionError(f"Kernel returned {len(produced)} outputs but the reference has {len(reference)}.")
    expected = [reconcile_output_layout(want, got.shape).to(got.device) for got, want in zip(produced, reference)]
    if compare == "softmax_partial" and own_cut(kernel):
        compare = "softmax_partial_folded"
    for got, want in zip(_comparable(produced, compare), _comparable(expected, compare)):
        torch.testing.assert_close(got.float(), want.float().to(got.device), rtol=tolerance.rtol,
                                   atol=tolerance.atol, equal_nan=tolerance.equal_nan)


def _check_kernel(kernel, *, graph=None, dtype=None, reference_cache_dir=None,
                  tolerance: Tolerance = DEFAULT_TOLERANCE, benchmark: BenchOptions | None = None):
    """A child's side: validate against the published reference (or one built here from
    ``graph`` and ``dtype``), then optionally time, all under one hold of the GPU lock.  Mean
    latency in ms, or None without ``benchmark``."""
    from . import reference as ref

    with _gpu_exec_guard():
        with _stage("validate"):
            if reference_cache_dir is None:
                inputs_by_name, expected, _ = ref.build_inputs_and_reference(graph, dtype)
                mode = compare_mode(graph)
            else:
                inputs_by_name, expected, mode = _ReferenceFile(reference_cache_dir).read()
            ordered = ref.order_inputs_for_kernel(inputs_by_name, kernel)
            _validate_kernel_outputs(kernel, ordered, expected, tolerance=tolerance, compare=mode)
        if benchmark is not None:
            with _stage("bench"):
                return benchmark_compiled_kernel(kernel, ordered, warmup_iters=benchmark.warmup,
                                                 profile_iters=benchmark.iters)
    return None


def _run_and_validate_kernel(kernel, **where):
    """``_check_kernel`` without timing; the kernel's source comes back."""
    where.pop("benchmark", None)
    _check_kernel(kernel, **where)
    return kernel.get_kernel_source()
