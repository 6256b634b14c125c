"""cleave_amd: an MI355X (gfx950) code-generation and runtime back end behind the Cleave API.

``cleave_amd.compile(fn, shapes=..., dtype=..., preset=...)`` on a ``@cleave_amd.jit`` program runs the
staged pipeline trace -> superoptimize -> schedule -> build -> evaluate; plans are instantiated
into hand-written HIP kernel templates, compiled with hiprtc for gfx950 and launched through
``libcleave_hip.so``.

Nothing heavy is imported until it is asked for: the public names below are resolved on first
attribute access (the top-level names are those of ``python/cleave/__init__.py``, so user code
only changes its import line).
"""

import importlib

__version__ = "0.1.0"

# home module (relative) -> the public names it provides
_PROVIDERS = {
    ".frontend": "Program trace jit JitFunction InputSpec OutputSpec",
    ".pipeline": ("compile superoptimize schedule_plans build evaluate load list_presets "
                  "SuperoptConfig ScheduleConfig EvalConfig GraphSet SearchedGraph Plan PlanSet BuildSet Report Kernel"),
    ".schedule": "search_tiling apply_tiling",
    ".codegen": "HipCodeGen",
    ".core.errors": "CleaveError",
    ".core.session": "Session",
}
_PACKAGES = "arch codegen core dynamic frontend ir lang pipeline runtime schedule".split()

_HOME = {name: module for module, names in _PROVIDERS.items() for name in names.split()}
__all__ = sorted(set(_HOME) | set(_PACKAGES))


def __getattr__(name):
    if name in _PACKAGES:
        value = importlib.import_module("." + name, __name__)
    elif name in _HOME:
        value = getattr(importlib.import_module(_HOME[name], __name__), name)
    else:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    globals()[name] = value          # the next access does not come back here
    return value


def __dir__():
    return list(__all__)
