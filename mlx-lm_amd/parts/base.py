"""Interfaces of the parts a model is put together from, and their registries.

A part takes its sizes and constants as constructor parameters, declares the
tensors it wants by name, and runs on a ``StepContext``.  It does not know
which model it is in.  Five kinds of part exist:

* ``Norm``             ``forward(ctx, x, rows=None, n_rows=None, lazy=False) -> y``;
                       with ``lazy`` it may return a ``NormedInput`` for a
                       consumer that set ``accepts_lazy_input``
* ``Mixer``            ``forward(ctx, x, residual, cache, writes_cache)`` adds
                       its output into ``residual``; ``cache_need()`` says
                       what cache slot it wants
* ``FeedForward``      ``forward(ctx, x, residual)`` adds into ``residual``
* ``PositionEncoding`` ``embedding_term(ctx)`` and ``rotate(ctx, q, k)``
* blocks               ``forward(ctx, h, cache, writes_cache)``; arrange two
                       norms, a mixer and a feed-forward

plus the token embedding and the output head.  ``x`` is ``[tokens, width]`` in
the compute dtype, ``residual``/``h`` the float32 residual stream.

A new kind is added with ``register_mixer`` and its siblings; a plan then
names it by its key.
"""

from dataclasses import dataclass
from typing import Dict, Tuple


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part wants: its shape and how it is kept on the device.

    ``role``: ``matrix`` tensors are cast to the compute dtype; ``vector``
    tensors (biases, norm scales) are kept in float32; ``int`` tables in int32.
    """

    shape: Tuple[int, ...]
    role: str = "matrix"


class Part:
    """Base of all parts."""

    def __init__(self, prefix=""):
        self.prefix = prefix

    def tensors(self) -> Dict[str, TensorSpec]:
        """Full tensor names (prefix included) to their specs."""
        return {}

    def load(self, tensors):
        """Receive the device tensors named in ``tensors()``."""

    def _name(self, local):
        return self.prefix + local


class Norm(Part):
    def forward(self, ctx, x, rows=None, n_rows=None, lazy=False):
        raise NotImplementedError


class Mixer(Part):
    def cache_need(self):
        """A ``CacheNeed``, a ``StateNeed`` or ``None``."""
        return None

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, ctx, x, residual):
        raise NotImplementedError


class PositionEncoding(Part):
    def embedding_term(self, ctx):
        """``(table, index)`` to add to the token embedding, or ``None``."""
        return None

    def rotate(self, ctx, q, k):
        """Encode positions into queries and keys in place (before the cache write)."""


class Block(Part):
    def forward(self, ctx, h, cache, writes_cache=True):
        raise NotImplementedError


NORMS = {}
MIXERS = {}
FEED_FORWARDS = {}
POSITION_ENCODINGS = {}
BLOCKS = {}
EMBEDDINGS = {}
HEADS = {}


def _registrar(table, what):
    def register(kind, cls):
        table[kind] = cls
        return cls

    register.__doc__ = f"Register a {what} class under the key ``kind``."
    return register


register_norm = _registrar(NORMS, "norm")
register_mixer = _registrar(MIXERS, "mixer")
register_feed_forward = _registrar(FEED_FORWARDS, "feed-forward")
register_position_encoding = _registrar(POSITION_ENCODINGS, "position encoding")
register_block = _registrar(BLOCKS, "block arrangement")
register_embedding = _registrar(EMBEDDINGS, "embedding")
register_head = _registrar(HEADS, "output head")


def build_part(table, what, spec, **extra):
    """Make the part that ``spec`` (a ``PartSpec``) describes."""
    try:
        cls = table[spec.kind]
    except KeyError:
        raise ValueError(f"unknown {what} kind '{spec.kind}' (known: {sorted(table)})") from None
    return cls(prefix=spec.prefix, **spec.params, **extra)
