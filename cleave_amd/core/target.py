"""The compilation target: always an AMD gfx950 device (MI355X).

The reference's ``Target`` (``python/cleave/core/target.py:7-106``) probes a CUDA device and
falls back to an offline description named by ``CLEAVE_TARGET_ARCH``.  Here the limits the
schedule search needs are a fixed description of gfx950, refined from the device through
the native library when a GPU is visible, so plans and source can be produced on a host
without one.
"""

from __future__ import annotations

import functools
import os


class Target:
    def __init__(self, kind: str = "hip"):
        if kind in ("cuda", "rocm"):  # the reference's spelling is accepted as an alias
            kind = "hip"
        if kind != "hip":
            raise ValueError(f"unsupported target kind {kind!r}; this back end only targets 'hip'")
        self.kind = kind

    @property
    def arch_name(self) -> str:
        return os.environ.get("CLEAVE_TARGET_ARCH", "gfx950")

    @functools.cached_property
    def arch(self):
        from ..arch import get_arch

        return get_arch(self.arch_name)

    def __repr__(self):
        return f"Target({self.kind!r}, arch={self.arch_name!r})"


@functools.lru_cache(maxsize=None)
def default_target(kind: str = "hip") -> Target:
    return Target(kind)


def current_target(kind: str = "hip") -> Target:
    from .session import active_session

    session = active_session()
    explicit = None if session is None else session.explicit_target
    return explicit if explicit is not None else default_target("hip")
