"""Position encodings."""
from typing import Dict, List

from .base import PositionEncoding, register_position
from .spec import ParamDecl


@register_position("learned")
class LearnedPositions(PositionEncoding):
    """A table with one row per position, added to the embedded tokens; row
    `position + offset` is read (reference: opt/model.py:232-244, where the
    offset is 2, and decoder.py:562-572)."""

    recordable = True

    def __init__(self, width: int, max_positions: int, offset: int = 0):
        self.width, self.max_positions, self.offset = width, max_positions, offset
        self.table = None

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        return [ParamDecl(prefix + ".weight", (self.max_positions + self.offset, self.width), "table")]

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.table = tensors[prefix + ".weight"]

    def at_input(self, x, positions, want_compute: bool):
        """x `[T, width]` (any float dtype) -> (float32 sum, compute-dtype copy or None)."""
        return self.ops.add_positions(x, positions, self.table, self.offset, self.dtype, want_compute)


@register_position("none")
class NoPositions(PositionEncoding):
    """No encoding at the input: the embedded tokens pass as they are."""

    recordable = True

    def __init__(self, **_):
        pass

    def at_input(self, x, positions, want_compute: bool):
        return self.ops.to_stream(x, self.dtype, want_compute)
