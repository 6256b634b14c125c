"""Structures -> stage graphs: one ``[main]`` graph, or ``[partial, combine]`` for a split.

The reference cuts a searched split structure at the reductions over the split axis
(``python/cleave/lower/split.py:386-717``) and lowers each side through TVM
(``python/cleave/lower/process.py:206-251``).  Here a stage is a recognised operator plus a
role; the partial's outputs and the combine's inputs are the family's partial buffers.
"""

from .stages import StageGraph, to_bundles, to_ir  # noqa: F401
