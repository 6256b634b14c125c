"""Exception hierarchy of the back end.

Mirrors the class names and base classes of the reference's
``python/cleave/core/errors.py:1-50`` so ``except`` clauses written against it keep
working: a validation failure is still an ``AssertionError``, a timeout still a
``TimeoutError``, a bad specification still a ``ValueError``.
"""


class CleaveError(Exception):
    """Root of every error this package raises on purpose."""


class SpecError(CleaveError, ValueError):
    """The user's program, shapes or options are inconsistent."""


class SuperoptError(CleaveError):
    """The graph-proposal stage failed."""


class LoweringRejected(CleaveError):
    """A proposed graph has no lowering onto a kernel family."""


class ScheduleRejected(CleaveError):
    """No launch plan exists for a lowered graph."""


class CodegenError(CleaveError):
    """Instantiating a kernel template failed (parent process, before any compile)."""


class CompileError(CleaveError):
    """hiprtc rejected the generated source, or the code object would not load."""


class LdsExceeded(CompileError):
    """The kernel asks for more LDS than a gfx950 workgroup may own (160 KiB)."""


# The reference's name for the same condition on its hardware.
SmemExceeded = LdsExceeded


class ValidationError(CleaveError, AssertionError):
    """A compiled candidate's output differs from the reference evaluation."""


class CandidateTimeout(CleaveError, TimeoutError):
    """A candidate exceeded its compile-and-run budget and its worker was killed."""


class WorkerCrash(CleaveError):
    """A candidate's worker process died before reporting."""


class PagingRefusal(CleaveError, AssertionError):
    """The paged access layer cannot wrap this plan."""


class BenchmarkError(CleaveError):
    """Timing a validated candidate failed."""


class BackendUnavailable(CleaveError, RuntimeError):
    """The native library is missing, or no GPU is visible for an operation that needs one."""
