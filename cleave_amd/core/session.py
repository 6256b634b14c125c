"""``Session``: target, cache root and parallelism scoped by a ``with`` block
(``python/cleave/core/session.py:22-64``)."""

from __future__ import annotations

import dataclasses
from contextvars import ContextVar
from pathlib import Path
from typing import Optional

from .settings import Settings
from .target import Target, default_target

_STACK: ContextVar[tuple] = ContextVar("cleave_amd_sessions", default=())


class Session:
    def __init__(self, target=None, cache_root=None, max_parallel: Optional[int] = None,
                 settings: Optional[Settings] = None):
        settings = settings or Settings.from_env()
        if cache_root is not None:
            settings = dataclasses.replace(settings, cache_root=Path(cache_root).expanduser())
        if max_parallel is not None and int(max_parallel) < 1:
            raise ValueError(f"max_parallel must be >= 1, got {max_parallel}")
        self.settings = settings
        self.explicit_target = Target(target) if isinstance(target, str) else target
        self.max_parallel = None if max_parallel is None else int(max_parallel)

    @property
    def target(self) -> Target:
        return self.explicit_target or default_target()

    @property
    def cache_root(self) -> Path:
        return Path(self.settings.cache_root)

    def __enter__(self):
        _STACK.set(_STACK.get() + (self,))
        return self

    def __exit__(self, *exc):
        stack = _STACK.get()
        if not stack or stack[-1] is not self:
            raise RuntimeError("Session exited out of order")
        _STACK.set(stack[:-1])

    def __repr__(self):
        return (f"Session(target={self.target!r}, cache_root={str(self.cache_root)!r}, "
                f"max_parallel={self.max_parallel})")


def active_session() -> Optional[Session]:
    stack = _STACK.get()
    return stack[-1] if stack else None


def current_session() -> Session:
    return active_session() or Session()
