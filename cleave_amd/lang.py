"""``import cleave_amd.lang as cl``: dims, dtypes, annotations and ops of the frontend
(the names of ``python/cleave/lang.py``)."""

from .frontend.composites import exp, matmul, max, mean, rms_norm, rsqrt, silu, sqrt, sum  # noqa: A004,F401
from .frontend.paged import PageTable, ScheduleHints, paged_gather, softmax  # noqa: F401
from .frontend.tensor import DType, Dim, Scalar, Split, Tensor, bf16, dims, f16, f32, i32  # noqa: F401

__all__ = [
    "DType", "Dim", "PageTable", "Scalar", "ScheduleHints", "Split", "Tensor", "Tolerance", "bf16",
    "dims", "exp", "f16", "f32", "i32", "matmul", "max", "mean", "paged_gather", "rms_norm", "rsqrt",
    "silu", "softmax", "sqrt", "sum", "workloads",
]


def __getattr__(name):
    if name == "Tolerance":
        from .runtime.validate import Tolerance

        return Tolerance
    if name == "workloads":
        from .frontend import paged

        return paged.workloads
    raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
