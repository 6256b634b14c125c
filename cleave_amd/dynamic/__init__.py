"""Dynamic (paged) attention operators: specs, access layer, references, workloads."""

from .registry import GATHER_TOLERANCE, OPERATORS, DynamicOperator  # noqa: F401
