"""Arrangements of norms, mixer and feed-forward in a layer."""

import ctypes

from ..ops import native
from .base import Block, register_block


class PreNormBlock(Block):
    """``h += mixer(norm1(h)); h += ffn(norm2(h))``.

    mlx_lm/models/gpt2.py:98-108.  The two sums happen inside the mixer's and
    the feed-forward's last matrix product, in float32.  Such a product may
    leave its sum into ``h`` pending (``ctx.pending``); the norm that reads
    ``h`` next adds it (``handles_pending``).  A mixer whose kernels leave CUs
    idle may have them read the weights that come after its own (the
    feed-forward's first).  The arrangement itself runs in the native host
    (``PreNormBlock`` in csrc/engine.hip); its parts may be native or Python.
    """

    PARTS = {"mixer_norm": "norm", "mixer": "mixer", "ffn_norm": "norm", "ffn": "feed_forward"}
    handles_pending = True

    def __init__(self, mixer_norm, mixer, ffn_norm, ffn, prefix=""):
        super().__init__(prefix)
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def cache_need(self):
        return self.mixer.cache_need()

    def make_native(self):
        return native.made(native.lib().eng_make_pre_norm_block(
            self.mixer_norm.native(), self.mixer.native(), self.ffn_norm.native(), self.ffn.native()),
            "pre-norm block")

    def forward(self, ctx, h, cache, writes_cache=True):
        hm = native.mat(h)
        with ctx.enter():
            rc = native.lib().eng_block_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(hm), cache.slot,
                                                int(bool(writes_cache)))
        native.check(rc, "pre-norm block")
        return h


register_block("pre_norm", PreNormBlock)
