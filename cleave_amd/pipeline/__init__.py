"""The staged compile pipeline: superoptimize -> schedule -> build -> evaluate -> ``Kernel``.

One stage per module; this file only gathers their public names (those a Cleave user imports
from ``cleave.pipeline``) into one namespace.
"""

from . import build as _build
from . import compile as _compile
from . import config as _config
from . import kernel as _kernel
from . import plans as _plans
from . import report as _report
from . import superopt as _superopt

_PUBLIC = {
    _superopt: ("GraphSet", "SearchedGraph", "superoptimize"),
    _plans: ("Plan", "PlanSet", "Refusal", "lower", "schedule"),
    _build: ("BuildSet", "BuiltKernel", "build", "evaluate"),
    _report: ("Failures", "Report", "Result", "VariantResult"),
    _kernel: ("Kernel", "load"),
    _compile: ("compile", "resolve_configs"),
    _config: ("PRESETS", "Preset", "SuperoptConfig", "ScheduleConfig", "EvalConfig", "auto_max_ops", "get_preset",
              "list_presets"),
}
for _module, _names in _PUBLIC.items():
    globals().update({_name: getattr(_module, _name) for _name in _names})
schedule_plans = _plans.schedule          # the name the top-level package exports the stage under

__all__ = sorted([name for names in _PUBLIC.values() for name in names] + ["schedule_plans"])
