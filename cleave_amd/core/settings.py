"""Process-wide knobs read from the environment.

The variable names are the ones a Cleave user already exports (``python/cleave/core/settings.py:34-52``,
``python/cleave/_cache_env.py:36-43``); how they are parsed is a small table here: one row per
knob, giving its variable, its parser and its default.
"""

from __future__ import annotations

import os
import tempfile
from pathlib import Path
from typing import Mapping, NamedTuple, Optional


def cache_root_from(env: Mapping[str, str]) -> Path:
    """Where caches go: ``CLEAVE_CACHE_ROOT`` as given; otherwise a ``cleave_cache`` folder under
    ``$SCRATCH`` when that is set, under the system's temporary directory when not."""
    for variable, leaf in (("CLEAVE_CACHE_ROOT", None), ("SCRATCH", "cleave_cache")):
        text = env.get(variable)
        if text:
            root = Path(text).expanduser()
            return root / leaf if leaf else root
    return Path(tempfile.gettempdir(), "cleave_cache")


def _limit(text: Optional[str], fallback):
    """A time span in seconds.  Unset, empty or unreadable text keeps the fallback; zero or a
    negative number means "no limit" (``None``)."""
    try:
        seconds = float(text) if text else None
    except ValueError:
        seconds = None
    if seconds is None:
        return fallback
    return seconds if seconds > 0 else None


_SWITCH_WORDS = {word: True for word in ("1", "true", "yes", "on")}
_SWITCH_WORDS.update({word: False for word in ("0", "false", "no", "off", "")})


def _switch(text: Optional[str], fallback: bool) -> bool:
    return fallback if text is None else _SWITCH_WORDS.get(text.strip().lower(), fallback)


def _seed(text: Optional[str], fallback):
    return fallback if text is None else int(text) % (1 << 32)


class _Knob(NamedTuple):
    variable: str
    parse: callable
    default: object


_KNOBS = {
    "compile_timeout_secs": _Knob("CLEAVE_COMPILE_AND_RUN_TIMEOUT_SECS", _limit, 300.0),
    "heartbeat_secs": _Knob("CLEAVE_COMPILE_PROGRESS_HEARTBEAT_SECS", _limit, 15.0),
    "progress_log": _Knob("COMPILATION_PROGRESS_LOG", _switch, False),
    "test_seed": _Knob("CLEAVE_TEST_SEED", _seed, None),
}


class Settings:
    """An immutable record of the knobs above plus the cache root.

    ``compile_timeout_secs``: wall-clock limit of one candidate's compile + validate + time
    (``None``: unlimited); ``heartbeat_secs``: spacing of progress lines; ``progress_log``: whether
    those lines are printed at all; ``test_seed``: 32-bit seed tests may pin; ``cache_root``: the
    folder ``runtime_root`` and ``persistent_root`` sit in.
    """

    __slots__ = (*_KNOBS, "cache_root")

    def __init__(self, **values):
        unknown = set(values) - set(self.__slots__)
        if unknown:
            raise TypeError(f"Settings has no field(s) {sorted(unknown)}")
        for name, knob in _KNOBS.items():
            object.__setattr__(self, name, values.get(name, knob.default))
        root = values.get("cache_root")
        object.__setattr__(self, "cache_root", None if root is None else Path(root))

    def __setattr__(self, name, value):
        raise AttributeError("Settings is immutable; use .replace(...)")

    def replace(self, **changes) -> "Settings":
        return Settings(**{**self.as_dict(), **changes})

    def as_dict(self) -> dict:
        return {name: getattr(self, name) for name in self.__slots__}

    def __eq__(self, other):
        return isinstance(other, Settings) and self.as_dict() == other.as_dict()

    def __hash__(self):
        return hash(tuple(self.as_dict().items()))

    def __repr__(self):
        return "Settings(" + ", ".join(f"{k}={v!r}" for k, v in self.as_dict().items()) + ")"

    @classmethod
    def from_env(cls, env: Optional[Mapping[str, str]] = None) -> "Settings":
        env = os.environ if env is None else env
        values = {name: knob.parse(env.get(knob.variable), knob.default) for name, knob in _KNOBS.items()}
        return cls(cache_root=cache_root_from(env), **values)

    # candidates' scratch files (references, lock files) / what survives between processes
    @property
    def runtime_root(self) -> Path:
        return self.cache_root / "runtime"

    @property
    def persistent_root(self) -> Path:
        return self.cache_root / "persistent"
