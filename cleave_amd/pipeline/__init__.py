"""Staged compile pipeline: superoptimize -> schedule -> build -> evaluate -> Kernel."""

from .build import BuildSet, BuiltKernel, build, evaluate
from .compile import compile, resolve_configs  # noqa: A004
from .config import (PRESETS, EvalConfig, Preset, ScheduleConfig, SuperoptConfig, auto_max_ops, get_preset,
                     list_presets)
from .kernel import Kernel, load
from .plans import Plan, PlanSet, Refusal, lower, schedule
from .report import Failures, Report, Result, VariantResult
from .superopt import GraphSet, SearchedGraph, superoptimize

schedule_plans = schedule

__all__ = ["BuildSet", "BuiltKernel", "EvalConfig", "Failures", "GraphSet", "Kernel", "PRESETS", "Plan", "PlanSet",
           "Preset", "Refusal", "Report", "Result", "ScheduleConfig", "SearchedGraph", "SuperoptConfig",
           "VariantResult", "auto_max_ops", "build", "compile", "evaluate", "get_preset", "list_presets", "load",
           "lower", "resolve_configs", "schedule", "schedule_plans", "superoptimize"]
