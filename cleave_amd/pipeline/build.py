"""The build and evaluate stages: plans in, checked and timed kernels out.

``build`` hands the tilings of a plan set to ``runtime.evaluate.run_candidates`` (source text is
generated in this process; compiling, validating and timing happen in child processes) and
attaches to every outcome its plan and, where source came back, a ``BuiltKernel``: the source
plus the call signature its manifest declares.  ``evaluate`` turns a finished build into a
``Report``.  What the stages mean is the reference's (``python/cleave/pipeline/build.py:148-180``);
a candidate must hold the strict 1e-2 / 1e-2 bound unless the config sets another.
"""

from __future__ import annotations

import time
from typing import NamedTuple

from .config import EvalConfig
from .plans import PlanSet
from .report import Report, Result, _Results

ENTRY = "main_kernel"


class KernelParam(NamedTuple):
    """One parameter of a generated kernel; ``role`` is input, output, scalar or scratch."""
    name: str
    dtype: str
    dims: tuple
    role: str

    @classmethod
    def of_manifest(cls, entry: dict) -> "KernelParam":
        return cls(entry["name"], entry["dtype"], tuple(entry["shape"]), entry["role"])


class BuiltKernel:
    """Generated source together with the call signature its manifest declares."""

    __slots__ = ("source", "entry", "params", "out_idx", "pass_configs", "dyn_dims", "plan")

    def __init__(self, source, entry=ENTRY, params=(), out_idx=(), pass_configs=None, dyn_dims=(), plan=None):
        self.source = source
        self.entry = entry
        self.params = tuple(params)
        self.out_idx = tuple(out_idx)
        self.pass_configs = dict(pass_configs or {})
        self.dyn_dims = tuple(dyn_dims)
        self.plan = plan

    def __repr__(self):
        listed = ", ".join(f"{p.role} {p.name}" for p in self.params)
        return f"BuiltKernel({self.entry}: {listed})"

    def having(self, role: str) -> list:
        return [p for p in self.params if p.role == role]

    inputs = property(lambda self: self.having("input"))
    outputs = property(lambda self: self.having("output"))

    # -- made from a plan's generated source ------------------------------------------------
    @classmethod
    def from_plan(cls, plan, source: str) -> "BuiltKernel":
        from ..codegen import parse_manifest

        declared = parse_manifest(source)
        return cls(source, entry=declared["launches"][0]["entry"],
                   params=map(KernelParam.of_manifest, declared["params"]), out_idx=declared["out_idx"],
                   dyn_dims=declared.get("dyn_dims") or (), plan=plan)

    # -- the ``kernel`` entry of a saved kernel.json -----------------------------------------
    def to_dict(self) -> dict:
        rows = [[p.name, p.dtype, list(p.dims), p.role] for p in self.params]
        return dict(entry=self.entry, out_idx=list(self.out_idx), dyn_dims=list(self.dyn_dims),
                    pass_configs=dict(self.pass_configs), params=rows)

    @classmethod
    def from_dict(cls, doc: dict, source: str, plan=None) -> "BuiltKernel":
        rows = doc.get("params") or ()
        return cls(source, entry=doc.get("entry", ENTRY),
                   params=(KernelParam(name, dtype, tuple(dims), role) for name, dtype, dims, role in rows),
                   out_idx=doc.get("out_idx") or (), pass_configs=doc.get("pass_configs"),
                   dyn_dims=doc.get("dyn_dims") or (), plan=plan)

    def compile(self):
        """The source compiled with hiprtc (loading and launching it then need a GPU)."""
        from ..runtime import compile as backend

        return backend._compile(backend._load_main_kernel_from_code(self.source), list(self.out_idx))


def resolve_tolerance(config):
    """``config.tolerance`` when set, else rtol = atol = 1e-2."""
    if config.tolerance:
        return config.tolerance
    from ..runtime.validate import STRICT_TOLERANCE

    return STRICT_TOLERANCE


def _described(plan, run):
    """The ``BuiltKernel`` of one outcome; None where no source came back or it carries no
    manifest (a test's stand-in build function, say)."""
    text = getattr(run, "code", None)
    if not text:
        return None
    try:
        return BuiltKernel.from_plan(plan, text)
    except Exception:  # noqa: BLE001 - whatever a foreign source makes the manifest parser raise
        return None


def built_kernels(plans, runs) -> list:
    return [_described(plan, run) for plan, run in zip(plans, runs)]


class BuildSet(_Results):
    """The outcomes of one ``build`` call, in plan order."""

    def __init__(self, results, plans: PlanSet | None = None, seconds: float = 0.0):
        self.plans, self.seconds = plans, seconds
        self.results = list(results)

    built = property(lambda self: self.correct)

    @property
    def kernels(self) -> list:
        return [outcome.kernel for outcome in self.results if outcome.kernel is not None]

    def __str__(self):
        return f"BuildSet: {len(self)} candidates, {len(self.correct)} ok, failures: {self.failures}"


def _element_type(plans) -> str:
    """The traced program's dtype name (the plan set's, else the first plan's; f16 when neither says)."""
    owner = getattr(plans, "program", None)
    if owner is None and len(plans):
        owner = plans[0].program
    return str(getattr(owner, "dtype", None) or "float16")


def _children_and_limit(workers, config):
    """How many child processes at once -- ``workers`` if given, else the current session's
    ``max_parallel`` if it sets one, else the config's -- and the seconds one candidate may take
    (the config's, else the session's; 0 switches the limit off)."""
    from ..core.session import current_session

    session = current_session()
    width = workers if workers is not None else (session.max_parallel or config.max_parallel)
    limit = config.timeout_s
    if limit is None:
        limit = session.settings.compile_timeout_secs or 0
    return width, limit


def build(plans, workers: int | None = None, *, config: EvalConfig | None = None, compiler_pass_options=None) -> BuildSet:
    """Check and time every plan."""
    from ..runtime.evaluate import run_candidates
    from ..runtime.validate import BenchOptions

    config = config or EvalConfig()
    width, limit = _children_and_limit(workers, config)
    queue = list(plans)
    started = time.perf_counter()
    outcomes = run_candidates([plan.tile for plan in queue], _element_type(plans), max_parallel=width,
                              timeout_s=limit, tolerance=resolve_tolerance(config),
                              benchmark=BenchOptions(config.warmup, config.iters),
                              compiler_pass_options=compiler_pass_options)
    rows = [Result(plan, run, _described(plan, run)) for plan, run in zip(queue, outcomes)]
    return BuildSet(rows, plans if isinstance(plans, PlanSet) else None, time.perf_counter() - started)


def evaluate(built, config: EvalConfig | None = None) -> Report:
    """The ``Report`` of a build; plans that are not built yet are built first with ``config``."""
    done = built if isinstance(built, BuildSet) else build(built, config=config)
    return Report(done.results, done.plans, {"build": done.seconds})
