"""Tracing frontend: ``@jit`` functions and the ``Program`` builder."""

from .jit import JitFunction, jit  # noqa: F401
from .paged import PagedAttention, PagedProgram, PageTable, ScheduleHints, is_paged, trace_paged  # noqa: F401
from .program import InputSpec, Op, OutputSpec, Program, grouped_matmul  # noqa: F401
from .tensor import DType, Dim, Scalar, Split, Tensor, bf16, dims, f16, f32, i32  # noqa: F401
from .trace import trace  # noqa: F401
