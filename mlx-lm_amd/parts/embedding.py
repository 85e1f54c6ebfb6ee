"""Token embedding: a row of the table for each token, written to the residual stream."""

from ..ops import kernels, native
from .base import Part, TensorSpec, register_embedding


class TokenEmbedding(Part):
    """``h[t] = table[ids[t]]``, plus a position term if the model has one.

    mlx_lm/models/gpt2.py:119-120,132.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, vocab_size, width, weight_name="weight", prefix=""):
        super().__init__(prefix)
        if vocab_size <= 0 or width <= 0:
            raise ValueError(f"embedding sizes must be positive, got {vocab_size} x {width}")
        self.vocab_size, self.width = vocab_size, width
        self.weight_name = self._name(weight_name)
        self.table = None

    def tensors(self):
        return {self.weight_name: TensorSpec((self.vocab_size, self.width), "matrix")}

    def load(self, tensors):
        self.table = tensors[self.weight_name]

    def reads_rows_of(self):
        """Tensors of which a step reads a row per token, not all."""
        return (self.weight_name,)

    native_kind = native.EMBEDDING

    def make_native(self):
        return native.made(native.lib().eng_make_token_embedding(
            self.table.data_ptr(), self.vocab_size, self.width, native.DT[self.table.dtype]), "token embedding")

    def forward(self, ctx, out, add=None):
        """Fill float32 ``out [tokens, width]``; ``add`` is ``(table, index)`` or ``None``."""
        if add is None:
            kernels.embed_gather_add(out, self.table, ctx.token_ids)
        else:
            kernels.embed_gather_add(out, self.table, ctx.token_ids, add[0], add[1])
        return out


register_embedding("token", TokenEmbedding)
