"""Position encodings."""

from ..ops import native
from .base import PositionEncoding, TensorSpec, register_position_encoding


class NoPositions(PositionEncoding):
    """Nothing is added and nothing is rotated."""

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, prefix=""):
        super().__init__(prefix)

    def make_native(self):
        return None  # no part at all


class LearnedPositions(PositionEncoding):
    """A learned table indexed by absolute position, added to the token embedding.

    ``h += wpe[arange(L) + offset]`` (mlx_lm/models/gpt2.py:121,137-144); the
    step's ``positions`` array already holds ``offset + i`` for every token.
    A position at or beyond the table's end is refused by the engine before
    anything runs (the reference does not check it).
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, max_positions, width, weight_name="weight", prefix=""):
        super().__init__(prefix)
        if max_positions <= 0:
            raise ValueError(f"max_positions must be positive, got {max_positions}")
        self.max_positions, self.width = max_positions, width
        self.weight_name = self._name(weight_name)
        self.table = None

    def tensors(self):
        return {self.weight_name: TensorSpec((self.max_positions, self.width), "matrix")}

    def load(self, tensors):
        self.table = tensors[self.weight_name]

    def reads_rows_of(self):
        """Tensors of which a step reads a row per token, not all."""
        return (self.weight_name,)

    def make_native(self):
        return native.made(native.lib().eng_make_learned_positions(
            self.table.data_ptr(), self.max_positions, self.width, native.DT[self.table.dtype]), "learned positions")

    def embedding_term(self, ctx):
        return self.table, ctx.positions


register_position_encoding("none", NoPositions)
register_position_encoding("learned", LearnedPositions)
