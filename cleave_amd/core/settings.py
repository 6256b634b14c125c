"""Environment-driven settings (same variables as ``python/cleave/core/settings.py:34-52``)."""

from __future__ import annotations

import os
import tempfile
from dataclasses import dataclass
from pathlib import Path
from typing import Mapping, Optional

_TRUE = {"1", "true", "yes", "on"}
_FALSE = {"0", "false", "no", "off", ""}


def cache_root_from(env: Mapping[str, str]) -> Path:
    """``CLEAVE_CACHE_ROOT``, else ``$SCRATCH/cleave_cache``, else the temp dir
    (``python/cleave/_cache_env.py:36-43``)."""
    explicit = env.get("CLEAVE_CACHE_ROOT")
    if explicit:
        return Path(explicit).expanduser()
    scratch = env.get("SCRATCH")
    base = Path(scratch).expanduser() if scratch else Path(tempfile.gettempdir())
    return base / "cleave_cache"


def _seconds(env, name, default):
    """A positive float, ``default`` when unset or unparsable, ``None`` (disabled) when <= 0."""
    text = env.get(name)
    if text in (None, ""):
        return default
    try:
        value = float(text)
    except ValueError:
        return default
    return value if value > 0 else None


def _flag(env, name, default=False):
    text = env.get(name)
    if text is None:
        return default
    text = text.strip().lower()
    if text in _TRUE:
        return True
    if text in _FALSE:
        return False
    return default


@dataclass(frozen=True)
class Settings:
    compile_timeout_secs: Optional[float] = 300.0
    heartbeat_secs: Optional[float] = 15.0
    progress_log: bool = False
    test_seed: Optional[int] = None
    cache_root: Optional[Path] = None

    @classmethod
    def from_env(cls, env: Optional[Mapping[str, str]] = None) -> "Settings":
        env = os.environ if env is None else env
        seed = env.get("CLEAVE_TEST_SEED")
        return cls(
            compile_timeout_secs=_seconds(env, "CLEAVE_COMPILE_AND_RUN_TIMEOUT_SECS", 300.0),
            heartbeat_secs=_seconds(env, "CLEAVE_COMPILE_PROGRESS_HEARTBEAT_SECS", 15.0),
            progress_log=_flag(env, "COMPILATION_PROGRESS_LOG"),
            test_seed=None if seed is None else int(seed) & 0xFFFFFFFF,
            cache_root=cache_root_from(env),
        )

    @property
    def runtime_root(self) -> Path:
        return Path(self.cache_root) / "runtime"

    @property
    def persistent_root(self) -> Path:
        return Path(self.cache_root) / "persistent"
