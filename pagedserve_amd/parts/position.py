"""Position encodings."""

from ..weights.loader import TABLE, ParamSpec
from .base import PositionEncoding
from .registry import register_position


@register_position("learned_absolute")
class LearnedAbsolutePositions(PositionEncoding):
    """A table row per position, added to the token embedding
    (src/model/paged_decoder.py:289,311-313).  Positions must lie in ``[0, max_positions)``
    (src/model/paged_decoder.py:519-522)."""

    graph_safe = True

    def __init__(self, width: int, dtype, max_positions: int):
        self.width = width
        self.dtype = dtype
        self.max_positions = max_positions

    def parameters(self):
        return {"table": ParamSpec((self.max_positions, self.width), TABLE)}

    def embedding_table(self):
        return self.table


@register_position("none")
class NoPositions(PositionEncoding):
    """Nothing is added and nothing is rotated."""

    graph_safe = True

    def __init__(self, width: int, dtype, max_positions: int = 0):
        self.width = width
        self.dtype = dtype
        self.max_positions = max_positions
