"""Light graph IR and operator recognition."""

from .families import Lowered, recognize  # noqa: F401
from .graph import ComputeOpNode, Graph, Node, OutputNode, PlaceHolderNode, to_ir  # noqa: F401
