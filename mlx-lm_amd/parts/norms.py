"""Norms over the width of the residual stream."""

from ..ops import kernels
from .base import Norm, TensorSpec, register_norm


class LayerNorm(Norm):
    """``(x - mean) / sqrt(var + eps) * weight + bias`` with biased variance.

    ``nn.LayerNorm(n_embd, eps=layer_norm_epsilon)`` in
    mlx_lm/models/gpt2.py:92-96,123.  Reads the float32 residual stream,
    computes in float32, writes the compute dtype.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded

    def __init__(self, width, eps, bias=True, prefix=""):
        super().__init__(prefix)
        self.width, self.eps, self.has_bias = width, float(eps), bias
        self.weight = self.bias = None

    def tensors(self):
        t = {self._name("weight"): TensorSpec((self.width,), "vector")}
        if self.has_bias:
            t[self._name("bias")] = TensorSpec((self.width,), "vector")
        return t

    def load(self, tensors):
        self.weight = tensors[self._name("weight")]
        self.bias = tensors[self._name("bias")] if self.has_bias else None

    def forward(self, ctx, x, rows=None, n_rows=None, lazy=False):
        if lazy and rows is None:
            # the consumer's first matrix product may norm the rows itself
            return kernels.NormedInput(ctx.scratch, x, self.weight, self.bias, self.eps, ctx.dtype)
        n = x.shape[0] if n_rows is None else n_rows
        out = ctx.scratch((n, self.width), ctx.dtype)
        kernels.layernorm(out, x, self.weight, self.bias, self.eps, rows=rows)
        return out


register_norm("layernorm", LayerNorm)
