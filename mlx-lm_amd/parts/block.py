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

    # A mixer's or feed-forward's last projection may leave its sum into ``h``
    # pending (``ctx.pending``); the norm that reads ``h`` next adds it.
    handles_pending = True

    def _normed(self, ctx, norm, h, consumer):
        if not getattr(norm, "settles_pending", False):
            ctx.pending.settle()
        lazy = getattr(consumer, "accepts_lazy_input", False)
        if getattr(norm, "reads_ahead", False):  # it takes the weights its result meets first
            return norm.forward(ctx, h, lazy=lazy, ahead=getattr(consumer, "first_weight", None))
        return norm.forward(ctx, h, lazy=lazy)

    def forward(self, ctx, h, cache, writes_cache=True):
        mark = ctx.scratch_mark()
        x = self._normed(ctx, self.mixer_norm, h, self.mixer)
        # (a mixer whose kernels leave CUs idle may have them read the weights that come after its own)
        ctx.read_ahead = getattr(self.ffn, "first_weight", None)
        self.mixer.forward(ctx, x, h, cache, writes_cache)
        ctx.read_ahead = None
        self.ffn.forward(ctx, self._normed(ctx, self.ffn_norm, h, self.ffn), h)
        ctx.scratch_release(mark)
        return h


register_block("pre_norm", PreNormBlock)
