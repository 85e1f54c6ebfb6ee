"""Norms over the width of the residual stream."""

import ctypes

from ..ops import kernels, native
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

    def make_native(self):
        return native.made(native.lib().eng_make_layernorm(self.width, self.eps, native.ptr(self.weight),
                                                           native.ptr(self.bias)), "layernorm")

    def forward(self, ctx, x, rows=None, n_rows=None, lazy=False, ahead=None):
        """``ahead``: the weights of the product that reads the result first, if its caller knows
        them: a kernel here that leaves most of the GPU idle reads them into the caches meanwhile.
        (The native twin does the work: a pending sum is added, fused with the norm where the
        kernel takes it; with ``lazy`` the norm may be left to the consumer's first product.)"""
        out = native.EngValue()
        xm = native.mat(x)
        with ctx.enter():
            rc = native.lib().eng_norm_forward(
                self.native(), ctypes.byref(ctx.c), ctypes.byref(xm), native.ptr(rows), int(n_rows or 0),
                int(bool(lazy)), ctypes.byref(ahead.c) if ahead is not None and hasattr(ahead, "c") else None,
                ctypes.byref(out))
        native.check(rc, "layernorm")
        if out.lazy:
            return kernels.NormedInput(ctx.scratch, x, self.weight, self.bias, self.eps, ctx.dtype)
        return ctx.tensor(out.m)


register_norm("layernorm", LayerNorm)
