"""A decoder-only model built from a plan: embedding, scheduled layers, final norm, head."""

from ..config.plan import CacheNeed, ModelPlan, StateNeed
from .base import (
    BLOCKS,
    EMBEDDINGS,
    FEED_FORWARDS,
    HEADS,
    MIXERS,
    NORMS,
    POSITION_ENCODINGS,
    build_part,
)


class DecoderModel:
    """The parts a ``ModelPlan`` names, and the forward pass over one step's tokens.

    The order of the reference's forward (mlx_lm/models/gpt2.py:125-151,
    161-168): embeddings, the layers, final norm, head; except that the norm
    and the head run only on the rows whose logits are wanted, and that the
    order of layers is the plan's schedule.
    """

    def __init__(self, plan: ModelPlan):
        self.plan = plan.validate()
        self.width, self.vocab_size = plan.width, plan.vocab_size
        self.max_positions = plan.max_positions
        self.embedding = build_part(EMBEDDINGS, "embedding", plan.embedding)
        self.embedding_positions = (
            build_part(POSITION_ENCODINGS, "position encoding", plan.embedding_positions)
            if plan.embedding_positions is not None
            else None
        )
        self.layers = []
        for spec in plan.layers:
            if spec.arrangement not in BLOCKS:
                raise ValueError(
                    f"unknown block arrangement '{spec.arrangement}' (known: {sorted(BLOCKS)})"
                )
            self.layers.append(
                BLOCKS[spec.arrangement](
                    build_part(NORMS, "norm", spec.mixer_norm),
                    build_part(MIXERS, "mixer", spec.mixer),
                    build_part(NORMS, "norm", spec.ffn_norm),
                    build_part(FEED_FORWARDS, "feed-forward", spec.ffn),
                )
            )
        self.schedule = list(plan.schedule)
        self.final_norm = build_part(NORMS, "norm", plan.final_norm)
        self.head = build_part(HEADS, "output head", plan.head)

    # -- tensors ------------------------------------------------------------

    def parts(self):
        yield self.embedding
        if self.embedding_positions is not None:
            yield self.embedding_positions
        for block in self.layers:
            yield from block.parts()
        yield self.final_norm
        yield self.head

    def expected_tensors(self):
        """Every tensor the model wants, by full name.  A name may be wanted by
        two parts (a tied head) if they agree on shape and role."""
        want = {}
        for part in self.parts():
            for name, spec in part.tensors().items():
                if name in want and want[name] != spec:
                    raise ValueError(f"tensor '{name}' is wanted as {want[name]} and as {spec}")
                want[name] = spec
        return want

    def load_tensors(self, tensors):
        for part in self.parts():
            part.load(tensors)

    # -- cache ---------------------------------------------------------------

    def cache_needs(self):
        """What each cache slot has to hold, from the mixer of the run that writes it."""
        needs = {}
        for run in self.schedule:
            need = self.layers[run.layer].mixer.cache_need()
            if run.writes_cache:
                needs[run.cache] = need
            elif needs[run.cache] != need:
                raise ValueError(
                    f"layer {run.layer} reads cache slot {run.cache} but wants {need}, "
                    f"the slot holds {needs[run.cache]}"
                )
        out = [needs[i] for i in range(len(needs))]
        for need in out:
            if need is not None and not isinstance(need, (CacheNeed, StateNeed)):
                raise TypeError(f"cache_need() must give a CacheNeed, a StateNeed or None, got {need!r}")
        return out

    # -- forward -------------------------------------------------------------

    def forward(self, ctx):
        """Run the step's tokens; returns float32 logits ``[n_wanted, vocab]`` or ``None``."""
        h = ctx.scratch((ctx.n_tokens, self.width), "float32")
        add = self.embedding_positions.embedding_term(ctx) if self.embedding_positions else None
        self.embedding.forward(ctx, h, add)
        pending = ctx.pending
        for run in self.schedule:
            block = self.layers[run.layer]
            # a block that does not know of pending sums gets the stream with everything added
            pending.allowed = getattr(block, "handles_pending", False)
            if not pending.allowed:
                pending.settle()
            block.forward(ctx, h, ctx.cache_view(run.cache), run.writes_cache)
        pending.allowed = False
        if ctx.n_wanted == 0 or not getattr(self.final_norm, "settles_pending", False):
            pending.settle()
        if ctx.n_wanted == 0:
            return None
        if ctx.wants_every_row:
            x = self.final_norm.forward(ctx, h)
        else:
            x = self.final_norm.forward(ctx, h, rows=ctx.wanted_rows, n_rows=ctx.n_wanted)
        logits = ctx.logits_out(ctx.n_wanted, self.vocab_size)
        self.head.forward(ctx, x, logits)
        return logits
