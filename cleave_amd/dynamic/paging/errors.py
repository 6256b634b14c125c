"""Refusals of the paged access layer (all ``PagingRefusal``, hence ``AssertionError``s)."""

from ...core.errors import PagingRefusal


class InvalidSpec(PagingRefusal):
    """The operator description contradicts itself."""


class NotDenseAttention(PagingRefusal):
    """The plan handed over is not a scheduled dense attention body."""


class UnsupportedTiling(PagingRefusal):
    """The layer cannot be built at this tiling."""
