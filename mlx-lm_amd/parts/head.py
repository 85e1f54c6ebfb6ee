"""Output heads: from the final normed rows to float32 logits."""

import ctypes

from ..ops import kernels, native
from .base import Part, TensorSpec, register_head, value_of


class LinearHead(Part):
    """``logits = x @ weight.T``, no bias.

    With ``weight_name`` set to the embedding table's name the head is tied:
    there is one buffer, used by both (``wte.as_linear``,
    mlx_lm/models/gpt2.py:167).
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, vocab_size, width, weight_name, prefix=""):
        super().__init__(prefix)
        self.vocab_size, self.width = vocab_size, width
        self.weight_name = weight_name  # a full name: the head may share another part's tensor
        self.weight = None

    def tensors(self):
        return {self.weight_name: TensorSpec((self.vocab_size, self.width), "matrix")}

    def load(self, tensors):
        self.weight = kernels.for_decode(tensors[self.weight_name])

    native_kind = native.HEAD

    def make_native(self):
        w = kernels.weight_struct(self.weight)
        return native.made(native.lib().eng_make_linear_head(ctypes.byref(w)), "linear head")

    def forward(self, ctx, x, out):
        v, o = value_of(x), native.mat(out)
        with ctx.enter():
            rc = native.lib().eng_head_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(v), ctypes.byref(o))
        native.check(rc, "linear head")
        return out


register_head("linear", LinearHead)
