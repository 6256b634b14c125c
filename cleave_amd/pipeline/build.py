"""The build and evaluate stages: plans in, checked and timed kernels out.

``build`` sends every plan's tiling through ``runtime.evaluate.run_candidates`` (source generated
here, compile + validate + time in child processes) and pairs each outcome with its plan and with
a ``BuiltKernel`` describing the generated source.  ``evaluate`` wraps a finished build into a
``Report``.  Stage semantics follow the reference (``python/cleave/pipeline/build.py:148-180``);
candidates are validated at the strict 1e-2 / 1e-2 bound unless the config brings its own.
"""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Any

from .config import EvalConfig
from .plans import PlanSet
from .report import Report, Result, _Results

ENTRY = "main_kernel"


@dataclass(frozen=True)
class KernelParam:
    name: str
    dtype: str
    dims: tuple
    role: str          # input | output | scalar | scratch


@dataclass(eq=False)
class BuiltKernel:
    """Generated source together with the call signature its manifest declares."""
    source: str = field(repr=False)
    entry: str = ENTRY
    params: tuple = ()
    out_idx: tuple = ()
    pass_configs: dict = field(default_factory=dict)
    dyn_dims: tuple = ()
    plan: Any = field(default=None, repr=False)

    def _with_role(self, role) -> list:
        return [p for p in self.params if p.role == role]

    @property
    def inputs(self) -> list:
        return self._with_role("input")

    @property
    def outputs(self) -> list:
        return self._with_role("output")

    @classmethod
    def from_plan(cls, plan, source: str) -> "BuiltKernel":
        from ..codegen import parse_manifest

        manifest = parse_manifest(source)
        signature = tuple(KernelParam(p["name"], p["dtype"], tuple(p["shape"]), p["role"]) for p in manifest["params"])
        return cls(source=source, entry=manifest["launches"][0]["entry"], params=signature,
                   out_idx=tuple(manifest["out_idx"]), dyn_dims=tuple(manifest.get("dyn_dims") or ()), plan=plan)

    def to_dict(self) -> dict:
        return {"entry": self.entry, "out_idx": list(self.out_idx), "dyn_dims": list(self.dyn_dims),
                "pass_configs": dict(self.pass_configs),
                "params": [[p.name, p.dtype, list(p.dims), p.role] for p in self.params]}

    @classmethod
    def from_dict(cls, doc: dict, source: str, plan=None) -> "BuiltKernel":
        signature = tuple(KernelParam(name, dtype, tuple(dims), role) for name, dtype, dims, role in doc.get("params") or ())
        return cls(source=source, entry=doc.get("entry", ENTRY), params=signature, out_idx=tuple(doc.get("out_idx") or ()),
                   pass_configs=dict(doc.get("pass_configs") or {}), dyn_dims=tuple(doc.get("dyn_dims") or ()), plan=plan)

    def compile(self):
        """The source compiled with hiprtc (loading and launching it then need a GPU)."""
        from ..runtime.compile import _compile, _load_main_kernel_from_code

        return _compile(_load_main_kernel_from_code(self.source), list(self.out_idx))


def resolve_tolerance(config):
    """``config.tolerance`` when set, else rtol = atol = 1e-2."""
    from ..runtime.validate import STRICT_TOLERANCE

    return config.tolerance if config.tolerance else STRICT_TOLERANCE


def built_kernels(plans, runs) -> list:
    """A ``BuiltKernel`` per plan, None where no source exists or it carries no manifest (a test's
    stand-in build function, say)."""
    described = []
    for plan, run in zip(plans, runs):
        kernel = None
        if getattr(run, "code", None):
            try:
                kernel = BuiltKernel.from_plan(plan, run.code)
            except Exception:  # noqa: BLE001
                kernel = None
        described.append(kernel)
    return described


class BuildSet(_Results):
    def __init__(self, results, plans: PlanSet | None = None, seconds: float = 0.0):
        self.results = list(results)
        self.plans = plans
        self.seconds = seconds

    @property
    def built(self) -> list:
        return self.correct

    @property
    def kernels(self) -> list:
        return [r.kernel for r in self.results if r.kernel is not None]

    def __str__(self):
        return f"BuildSet: {len(self)} candidates, {len(self.correct)} ok, failures: {self.failures}"


def _dtype_of(plans) -> str:
    program = getattr(plans, "program", None)
    if program is None and len(plans):
        program = plans[0].program
    return str(getattr(program, "dtype", None) or "float16")


def build(plans, workers: int | None = None, *, config: EvalConfig | None = None, compiler_pass_options=None) -> BuildSet:
    """Check and time every plan.  Children at once: ``workers`` if given, else the current
    session's ``max_parallel`` if it sets one, else the config's."""
    from ..core.session import current_session
    from ..runtime.evaluate import run_candidates
    from ..runtime.validate import BenchOptions

    config = config or EvalConfig()
    session = current_session()
    width = workers
    if width is None:
        width = session.max_parallel or config.max_parallel
    limit = config.timeout_s
    if limit is None:
        limit = session.settings.compile_timeout_secs or 0      # 0 switches the limit off
    todo = list(plans)
    began = time.perf_counter()
    runs = run_candidates([plan.tile for plan in todo], _dtype_of(plans), max_parallel=width,
                          tolerance=resolve_tolerance(config), timeout_s=limit,
                          compiler_pass_options=compiler_pass_options,
                          benchmark=BenchOptions(config.warmup, config.iters))
    results = [Result(plan, run, kernel) for plan, run, kernel in zip(todo, runs, built_kernels(todo, runs))]
    return BuildSet(results, plans if isinstance(plans, PlanSet) else None, time.perf_counter() - began)


def evaluate(built, config: EvalConfig | None = None) -> Report:
    """The ``Report`` of a build; plans that are not built yet are built first with ``config``."""
    if not isinstance(built, BuildSet):
        built = build(built, config=config)
    return Report(built.results, built.plans, {"build": built.seconds})
