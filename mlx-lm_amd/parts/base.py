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
* blocks               ``forward(ctx, h, cache, writes_cache)``; an arrangement
                       names its parts and their families in ``PARTS``

plus the token embedding and the output head.  ``x`` is ``[tokens, width]`` in
the compute dtype, ``residual``/``h`` the float32 residual stream.

A new kind is added with ``register_mixer`` and its siblings; a plan then
names it by its key.

A step's launches are issued by the native host (``csrc/engine.hip``), which
walks a tree of native parts.  A built-in part describes itself to it
(``make_native``: its sizes, constants and device pointers) and its Python
``forward`` only calls its native twin, for a part used alone.  A part that
defines ``forward`` in Python and no ``make_native`` is wrapped as a callback
part: the native walk calls its ``forward`` where its turn comes, with torch
tensors over the walk's own memory.

A part may ask the packer for integer arrays of its own for every step:
``step_arrays_key`` (a name that parts sharing the same arrays share),
``step_array_names`` and ``step_arrays(batch) -> {name: list of int | int}``
(``batch``: a ``HostBatch``); they arrive as ``ctx.array(f"{key}.{name}")`` and,
for native parts, in ``EngCtx.arrays`` from the id ``native.array_ids`` gave.
"""

import ctypes
from dataclasses import dataclass
from typing import Dict, Tuple

from ..ops import native


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

    native_kind = None  # which kind of native part stands for it (native.NORM, ...)
    _native = None

    def __init__(self, prefix=""):
        self.prefix = prefix

    def native(self):
        """The handle of this part's native twin, made at first use (after ``load``)."""
        if self._native is None:
            self._native = self.make_native()
        return self._native

    def make_native(self):
        """By default a callback part: the native walk calls this object's Python methods."""
        if self.native_kind is None:
            raise TypeError(f"{type(self).__name__} cannot stand in a native model")
        flags = 0
        if getattr(self, "settles_pending", False):
            flags |= native.SETTLES_PENDING
        self._python_id = native.register_python_part(self)
        return native.made(native.lib().eng_make_callback(self.native_kind, self._python_id, flags),
                           type(self).__name__)

    def __del__(self):
        handle, self._native = self._native, None
        if handle:
            try:
                native.lib().eng_free(handle)
            except Exception:  # noqa: BLE001 (the interpreter may be shutting down)
                pass

    def tensors(self) -> Dict[str, TensorSpec]:
        """Full tensor names (prefix included) to their specs."""
        return {}

    def load(self, tensors):
        """Receive the device tensors named in ``tensors()``."""

    def _name(self, local):
        return self.prefix + local


def value_of(x):
    """The native description of a mixer's or feed-forward's input: a tensor, or a norm not computed yet."""
    from ..ops.kernels import NormedInput

    v = native.EngValue()
    if isinstance(x, NormedInput):
        v.lazy, v.ldx = 1, x.x.stride(0)
        v.m = native.EngMat(None, x.shape[0], x.shape[1], x.shape[1], native.DT[x.dtype])
        v.x, v.gamma, v.beta, v.eps = x.x.data_ptr(), native.ptr(x.gamma), native.ptr(x.beta), x.eps
    else:
        v.m = native.mat(x)
    return v


class Norm(Part):
    native_kind = native.NORM

    def forward(self, ctx, x, rows=None, n_rows=None, lazy=False):
        raise NotImplementedError


class Mixer(Part):
    native_kind = native.MIXER

    def cache_need(self):
        """A ``CacheNeed``, a ``StateNeed`` or ``None``."""
        return None

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        raise NotImplementedError


class FeedForward(Part):
    native_kind = native.FFN

    def forward(self, ctx, x, residual):
        raise NotImplementedError


class PositionEncoding(Part):
    native_kind = native.POSITION

    def embedding_term(self, ctx):
        """``(table, index)`` to add to the token embedding, or ``None``."""
        return None

    def rotate(self, ctx, q, k):
        """Encode positions into queries and keys in place (before the cache write)."""


class Block(Part):
    """An arrangement of parts in a layer.  ``PARTS`` names them and their families
    (``norm``, ``mixer``, ``feed_forward``, ``position_encoding``); the constructor gets the
    built parts under those names.  ``cache_need()`` is that of the part that keeps a cache."""

    native_kind = native.BLOCK
    PARTS: Dict[str, str] = {}

    def parts(self):
        return ()

    def cache_need(self):
        return None

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


FAMILIES = {
    "norm": (NORMS, "norm"),
    "mixer": (MIXERS, "mixer"),
    "feed_forward": (FEED_FORWARDS, "feed-forward"),
    "position_encoding": (POSITION_ENCODINGS, "position encoding"),
}


def build_part(table, what, spec, **extra):
    """Make the part that ``spec`` (a ``PartSpec``) describes."""
    try:
        cls = table[spec.kind]
    except KeyError:
        raise ValueError(f"unknown {what} kind '{spec.kind}' (known: {sorted(table)})") from None
    return cls(prefix=spec.prefix, **spec.params, **extra)
