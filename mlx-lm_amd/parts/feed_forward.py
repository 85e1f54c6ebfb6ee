"""Feed-forward parts."""

import ctypes

import torch

from ..ops import kernels, native
from .base import FeedForward, TensorSpec, register_feed_forward, value_of

_TANH_GELU = ("gelu_new", "gelu_pytorch_tanh", "gelu_tanh", "gelu_approx")


class GeluMLP(FeedForward):
    """``residual += c_proj(gelu_tanh(c_fc(x)))``, dense, with biases.

    mlx_lm/models/gpt2.py:71-80; the activation and the bias add are fused
    into the first product, the residual add into the second.
    """

    graph_safe = True  # launches kernels only: a step of such parts can be recorded
    accepts_lazy_input = True  # the first product can norm its input itself

    def __init__(self, width, inner, activation="gelu_new", prefix=""):
        super().__init__(prefix)
        if activation not in _TANH_GELU:
            raise ValueError(
                f"activation '{activation}' is not implemented (only the tanh GELU: {_TANH_GELU})"
            )
        if width % 8:
            raise ValueError(f"the feed-forward's width must be a multiple of 8, got {width}")
        if inner <= 0:
            raise ValueError(f"the feed-forward's inner size must be positive, got {inner}")
        self.width, self.inner = width, inner
        # The products want a multiple of 8 along K.  Inner features beyond ``inner`` get zero
        # weights and a zero bias: gelu(0) = 0 meets zero columns, so the sum is unchanged.
        self.inner_padded = (inner + 7) // 8 * 8
        self.fc_w = self.fc_b = self.proj_w = self.proj_b = None

    def tensors(self):
        n = self._name
        return {
            n("c_fc.weight"): TensorSpec((self.inner, self.width), "matrix"),
            n("c_fc.bias"): TensorSpec((self.inner,), "vector"),
            n("c_proj.weight"): TensorSpec((self.width, self.inner), "matrix"),
            n("c_proj.bias"): TensorSpec((self.width,), "vector"),
        }

    def load(self, tensors):
        n = self._name
        self.fc_w, self.fc_b = tensors[n("c_fc.weight")], tensors[n("c_fc.bias")]
        self.proj_w, self.proj_b = tensors[n("c_proj.weight")], tensors[n("c_proj.bias")]
        pad = self.inner_padded - self.inner
        if pad:
            self.fc_w = torch.cat([self.fc_w, self.fc_w.new_zeros(pad, self.width)]).contiguous()
            self.fc_b = torch.cat([self.fc_b, self.fc_b.new_zeros(pad)]).contiguous()
            self.proj_w = torch.cat([self.proj_w, self.proj_w.new_zeros(self.width, pad)], dim=1).contiguous()
        self.fc_w, self.proj_w = kernels.for_decode(self.fc_w), kernels.for_decode(self.proj_w)
        self.first_weight = self.fc_w  # what the first product reads

    def make_native(self):
        fc_w, proj_w = kernels.weight_struct(self.fc_w), kernels.weight_struct(self.proj_w)
        return native.made(native.lib().eng_make_gelu_mlp(
            self.width, self.inner_padded, ctypes.byref(fc_w), native.ptr(self.fc_b), ctypes.byref(proj_w),
            native.ptr(self.proj_b)), "gelu_mlp")

    def forward(self, ctx, x, residual):
        v, r = value_of(x), native.mat(residual)
        with ctx.enter():
            rc = native.lib().eng_ffn_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(v), ctypes.byref(r))
        native.check(rc, "gelu_mlp")


register_feed_forward("gelu_mlp", GeluMLP)
