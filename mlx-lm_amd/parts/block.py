"""Arrangements of norms, mixer and feed-forward in a layer."""

from .base import Block, register_block


class PreNormBlock(Block):
    """``h += mixer(norm1(h)); h += ffn(norm2(h))``.

    mlx_lm/models/gpt2.py:98-108.  The two sums happen inside the mixer's and
    the feed-forward's last matrix product, in float32.
    """

    def __init__(self, mixer_norm, mixer, ffn_norm, ffn, prefix=""):
        super().__init__(prefix)
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn)

    def forward(self, ctx, h, cache, writes_cache=True):
        mark = ctx.scratch_mark()
        lazy = getattr(self.mixer, "accepts_lazy_input", False)
        self.mixer.forward(ctx, self.mixer_norm.forward(ctx, h, lazy=lazy), h, cache, writes_cache)
        lazy = getattr(self.ffn, "accepts_lazy_input", False)
        self.ffn.forward(ctx, self.ffn_norm.forward(ctx, h, lazy=lazy), h)
        ctx.scratch_release(mark)
        return h


register_block("pre_norm", PreNormBlock)
