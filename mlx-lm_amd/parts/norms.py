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

    settles_pending = True  # adds a sum that is pending on ``x`` before (or while) it norms the rows
    reads_ahead = True  # ``forward`` takes ``ahead``, the weights that its result meets first

    def forward(self, ctx, x, rows=None, n_rows=None, lazy=False, ahead=None):
        """``ahead``: the weights of the product that reads the result first, if its caller knows
        them: a kernel here that leaves most of the GPU idle reads them into the caches meanwhile."""
        pending = ctx.pending
        if pending.waits_on(x):
            if rows is None and pending.can_norm(x):
                # the last projection split its sum: add the parts and norm the new rows in one kernel
                out = ctx.scratch((x.shape[0], self.width), ctx.dtype)
                if ahead is not None and not kernels.read_ahead_pays(ahead, x.shape[0]):
                    ahead = None
                pending.settle_normed(out, self.weight, self.bias, self.eps, ahead=ahead)
                return out
            pending.settle()
        if lazy and rows is None:
            # the consumer's first matrix product may norm the rows itself
            return kernels.NormedInput(ctx.scratch, x, self.weight, self.bias, self.eps, ctx.dtype)
        n = x.shape[0] if n_rows is None else n_rows
        out = ctx.scratch((n, self.width), ctx.dtype)
        kernels.layernorm(out, x, self.weight, self.bias, self.eps, rows=rows)
        return out


register_norm("layernorm", LayerNorm)
