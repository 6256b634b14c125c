"""Stages 3-4: build (codegen, then compile + validate + time in workers) and evaluate
(``python/cleave/pipeline/build.py:25-180``)."""

from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Any, Sequence

from .config import EvalConfig
from .plans import Plan, PlanSet
from .report import Report, Result, _Results

ENTRY = "main_kernel"


@dataclass(frozen=True)
class KernelParam:
    name: str
    dtype: str
    dims: tuple
    role: str      # "input" | "output" (| "scalar" | "scratch" for dynamic kernels)


@dataclass(eq=False)
class BuiltKernel:
    """One generated HIP kernel: its source plus the call signature its manifest declares."""

    source: str = field(repr=False)
    entry: str = ENTRY
    params: tuple = ()
    out_idx: tuple = ()
    pass_configs: dict = field(default_factory=dict)
    dyn_dims: tuple = ()
    plan: Any = field(default=None, repr=False)

    @property
    def inputs(self) -> list:
        return [p for p in self.params if p.role == "input"]

    @property
    def outputs(self) -> list:
        return [p for p in self.params if p.role == "output"]

    @classmethod
    def from_plan(cls, plan, source: str) -> "BuiltKernel":
        from ..codegen import parse_manifest

        m = parse_manifest(source)
        params = tuple(KernelParam(p["name"], p["dtype"], tuple(p["shape"]), p["role"]) for p in m["params"])
        return cls(source, m["launches"][0]["entry"], params, tuple(m["out_idx"]), {}, tuple(m.get("dyn_dims", ())), plan)

    def to_dict(self) -> dict:
        return {"entry": self.entry, "params": [[p.name, p.dtype, list(p.dims), p.role] for p in self.params],
                "out_idx": list(self.out_idx), "pass_configs": dict(self.pass_configs), "dyn_dims": list(self.dyn_dims)}

    @classmethod
    def from_dict(cls, d: dict, source: str, plan=None) -> "BuiltKernel":
        params = tuple(KernelParam(n, t, tuple(s), r) for n, t, s, r in d.get("params", ()))
        return cls(source, d.get("entry", ENTRY), params, tuple(d.get("out_idx", ())),
                   dict(d.get("pass_configs") or {}), tuple(d.get("dyn_dims", ())), plan)

    def compile(self):
        """hiprtc-compile the source (loading and launching need a GPU)."""
        from ..runtime.compile import _compile, _load_main_kernel_from_code

        return _compile(_load_main_kernel_from_code(self.source), list(self.out_idx))


def resolve_tolerance(config):
    """The bound candidates are validated against: the config's, else the strict 1e-2 / 1e-2."""
    from ..runtime.validate import STRICT_TOLERANCE

    return config.tolerance or STRICT_TOLERANCE


def built_kernels(plans: Sequence[Plan], runs) -> list:
    out = []
    for plan, run in zip(plans, runs):
        code = getattr(run, "code", None)
        try:
            out.append(BuiltKernel.from_plan(plan, code) if code else None)
        except Exception:  # noqa: BLE001 - injected fakes produce source without a manifest
            out.append(None)
    return out


class BuildSet(_Results):
    def __init__(self, results, plans: PlanSet | None = None, seconds: float = 0.0):
        self.results, self.plans, self.seconds = list(results), plans, seconds

    @property
    def built(self) -> list:
        return self.correct

    @property
    def kernels(self) -> list:
        return [r.kernel for r in self.results if r.kernel is not None]

    def __str__(self):
        return f"BuildSet: {len(self)} candidates, {len(self.correct)} ok, failures: {self.failures}"


def _program_dtype(plans) -> str:
    program = getattr(plans, "program", None)
    if program is None and len(plans):
        program = plans[0].program
    return str(getattr(program, "dtype", None) or "float16")


def build(plans, workers: int | None = None, *, config: EvalConfig | None = None,
          compiler_pass_options=None) -> BuildSet:
    """Compile, validate and time every plan (each in a worker, so a fault costs one candidate).
    Parallelism: ``workers``, else the active ``Session.max_parallel``, else ``config``."""
    from ..core.session import current_session
    from ..runtime.evaluate import run_candidates
    from ..runtime.validate import BenchOptions

    config = config or EvalConfig()
    session = current_session()
    timeout = config.timeout_s
    if timeout is None:
        timeout = session.settings.compile_timeout_secs or 0
    plan_list = list(plans)
    t0 = time.perf_counter()
    parallel = workers if workers is not None else (session.max_parallel or config.max_parallel)
    runs = run_candidates([p.tile for p in plan_list], _program_dtype(plans), max_parallel=parallel,
                          tolerance=resolve_tolerance(config), timeout_s=timeout,
                          compiler_pass_options=compiler_pass_options,
                          benchmark=BenchOptions(config.warmup, config.iters))
    kernels = built_kernels(plan_list, runs)
    results = [Result(p, r, k) for p, r, k in zip(plan_list, runs, kernels)]
    return BuildSet(results, plans if isinstance(plans, PlanSet) else None, time.perf_counter() - t0)


def evaluate(built, config: EvalConfig | None = None) -> Report:
    """The ``Report`` of a ``BuildSet`` (plans are built first, with ``config``)."""
    if not isinstance(built, BuildSet):
        built = build(built, config=config)
    return Report(built.results, built.plans, {"build": built.seconds})
