"""``Session``: a ``with`` block that scopes the target, the cache root and the search width.

Stands in for ``python/cleave/core/session.py:22-64`` (same constructor arguments and attributes).
Sessions nest; each is a link in a chain held by one context variable, so threads and asyncio
tasks each see their own innermost session.
"""

from __future__ import annotations

from contextvars import ContextVar
from pathlib import Path
from typing import Optional

from .settings import Settings
from .target import Target, default_target

# innermost entered session of the current context (None outside every ``with Session(...)``)
_INNERMOST: ContextVar[Optional["Session"]] = ContextVar("cleave_amd_session", default=None)


def _as_target(value):
    return Target(value) if isinstance(value, str) else value


def _as_width(value):
    if value is None:
        return None
    width = int(value)
    if width < 1:
        raise ValueError(f"max_parallel must be >= 1, got {value}")
    return width


class Session:
    """``target``: a ``Target`` or its name (default: detected); ``cache_root``: overrides the
    environment's; ``max_parallel``: candidates compiled / validated side by side (default: the
    evaluation config's); ``settings``: a ready ``Settings`` instead of the environment's."""

    def __init__(self, target=None, cache_root=None, max_parallel: Optional[int] = None,
                 settings: Optional[Settings] = None):
        self.max_parallel = _as_width(max_parallel)
        self.explicit_target = _as_target(target)
        base = Settings.from_env() if settings is None else settings
        self.settings = base if cache_root is None else base.replace(cache_root=Path(cache_root).expanduser())
        self._outer = None
        self._entered = False

    target = property(lambda self: self.explicit_target or default_target())
    cache_root = property(lambda self: Path(self.settings.cache_root))

    def __enter__(self):
        if self._entered:
            raise RuntimeError("this Session is already entered")
        self._outer, self._entered = _INNERMOST.get(), True
        _INNERMOST.set(self)
        return self

    def __exit__(self, *exc):
        if _INNERMOST.get() is not self:
            raise RuntimeError("Session exited out of order")
        _INNERMOST.set(self._outer)
        self._outer, self._entered = None, False

    def __repr__(self):
        fields = {"target": self.target, "cache_root": str(self.cache_root), "max_parallel": self.max_parallel}
        return "Session(" + ", ".join(f"{k}={v!r}" for k, v in fields.items()) + ")"


def active_session() -> Optional[Session]:
    """The innermost entered session, or ``None``."""
    return _INNERMOST.get()


def current_session() -> Session:
    """The innermost entered session, or a fresh one built from the environment."""
    return _INNERMOST.get() or Session()
