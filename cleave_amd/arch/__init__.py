"""Hardware description used by the schedule search."""

from .gfx950 import GFX950, Arch, get_arch  # noqa: F401
