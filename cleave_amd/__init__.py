"""cleave_amd: an MI355X (gfx950) code-generation and runtime back end behind the Cleave API.

``cleave_amd.compile(fn, shapes=..., dtype=..., preset=...)`` on a ``@cleave_amd.jit`` program
follows the same staged pipeline as the reference (trace -> superoptimize -> schedule ->
build -> evaluate), but plans are instantiated into hand-written HIP kernel templates,
compiled with hiprtc for gfx950 and launched through ``libcleave_hip.so``.
"""

from importlib import import_module

__version__ = "0.1.0"

_LAZY = {
    "HipCodeGen": ".codegen",
    "search_tiling": ".schedule",
    "apply_tiling": ".schedule",
    "Program": ".frontend",
    "trace": ".frontend",
    "jit": ".frontend",
    "JitFunction": ".frontend",
    "InputSpec": ".frontend",
    "OutputSpec": ".frontend",
    "compile": ".pipeline",
    "superoptimize": ".pipeline",
    "schedule_plans": ".pipeline",
    "build": ".pipeline",
    "evaluate": ".pipeline",
    "load": ".pipeline",
    "list_presets": ".pipeline",
    "SuperoptConfig": ".pipeline",
    "ScheduleConfig": ".pipeline",
    "EvalConfig": ".pipeline",
    "GraphSet": ".pipeline",
    "SearchedGraph": ".pipeline",
    "Plan": ".pipeline",
    "PlanSet": ".pipeline",
    "BuildSet": ".pipeline",
    "Report": ".pipeline",
    "Kernel": ".pipeline",
    "CleaveError": ".core.errors",
    "Session": ".core.session",
}
_SUBMODULES = {"core", "arch", "ir", "schedule", "codegen", "runtime", "dynamic", "frontend", "pipeline", "lang"}

__all__ = sorted([*_LAZY, *_SUBMODULES])


def __getattr__(name: str):
    if name in _SUBMODULES:
        return import_module(f".{name}", __name__)
    if name in _LAZY:
        return getattr(import_module(_LAZY[name], __name__), name)
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")


def __dir__():
    return __all__
