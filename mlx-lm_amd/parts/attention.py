"""Causal self-attention over the paged cache."""

import ctypes

from ..config.plan import CacheNeed
from ..ops import kernels, native
from .base import POSITION_ENCODINGS, Mixer, TensorSpec, build_part, register_mixer, value_of

ROW_KERNEL_MAX_Q = 4  # requests with at most this many tokens in a step take the row kernels
# (how many queries a tile of the general kernel and of the matrix-core prefill kernel holds is the
# kernels' own business: ``kernels.attn_tile_sizes()`` asks their libraries)


class CausalSelfAttention(Mixer):
    """Fused q/k/v projection, cache write, attention, output projection.

    ``residual += c_proj(attend(split(c_attn(x))))`` as in
    mlx_lm/models/gpt2.py:44-68: the fused projection gives queries, keys and
    values in that order, head ``h`` taking columns ``h*head_dim ..``; keys and
    values of this step's tokens go to their pages
    (mlx_lm/models/cache.py:333-355) and every query attends, through its
    request's block table, to the keys at or before its own position
    (mlx_lm/models/base.py:24-35,132-139).  ``n_kv_heads`` below ``n_heads``
    shares each key head among a group of query heads; ``window`` limits a
    query to the last ``window`` keys; ``position`` may rotate queries and keys
    before the cache write.
    """


    def __init__(self, width, n_heads, head_dim, n_kv_heads=None, scale=None, bias=True, window=0,
                 position=None, qkv_name="c_attn", out_name="c_proj", prefix=""):
        super().__init__(prefix)
        n_kv_heads = n_heads if n_kv_heads is None else n_kv_heads
        if n_heads <= 0 or n_kv_heads <= 0 or n_heads % n_kv_heads:
            raise ValueError(f"{n_heads} query heads cannot be grouped over {n_kv_heads} key heads")
        if head_dim % 16 or not (16 <= head_dim <= 256):
            raise ValueError(f"head_dim {head_dim} must be a multiple of 16 between 16 and 256")
        if width % 8:
            raise ValueError(f"width {width} must be a multiple of 8")
        if window < 0:
            raise ValueError(f"window {window} must not be negative")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.scale = float(scale) if scale is not None else head_dim**-0.5
        self.has_bias, self.window = bias, int(window)
        self.q_width = n_heads * head_dim
        self.kv_width = n_kv_heads * head_dim
        self.qkv_name, self.out_name = qkv_name, out_name
        self.position = (
            build_part(POSITION_ENCODINGS, "position encoding", position) if position is not None else None
        )
        self.qkv_w = self.qkv_b = self.out_w = self.out_b = None
        self.accepts_lazy_input = True  # the fused projection can norm its input itself
        # launches kernels only (a step of such parts can be recorded), unless the position hook does more
        self.graph_safe = self.position is None or getattr(self.position, "graph_safe", False)

    def cache_need(self):
        return CacheNeed(self.n_kv_heads, self.head_dim, self.window)

    def tensors(self):
        n = self._name
        t = {
            n(self.qkv_name + ".weight"): TensorSpec((self.q_width + 2 * self.kv_width, self.width), "matrix"),
            n(self.out_name + ".weight"): TensorSpec((self.width, self.q_width), "matrix"),
        }
        if self.has_bias:
            t[n(self.qkv_name + ".bias")] = TensorSpec((self.q_width + 2 * self.kv_width,), "vector")
            t[n(self.out_name + ".bias")] = TensorSpec((self.width,), "vector")
        if self.position is not None:
            t.update(self.position.tensors())
        return t

    def load(self, tensors):
        n = self._name
        self.qkv_w = tensors[n(self.qkv_name + ".weight")]
        self.out_w = tensors[n(self.out_name + ".weight")]
        if self.has_bias:
            self.qkv_b = tensors[n(self.qkv_name + ".bias")]
            self.out_b = tensors[n(self.out_name + ".bias")]
        self.qkv_w, self.out_w = kernels.for_decode(self.qkv_w), kernels.for_decode(self.out_w)
        self.first_weight = self.qkv_w  # what the mixer's first product reads
        if self.position is not None:
            self.position.load(tensors)

    # -- the step arrays this part asks the packer for ---------------------------

    step_arrays_key = "attention"
    step_array_names = ("tiles", "rows", "all_tiles", "big_tiles", "max_row_context", "rows_are_requests")

    @staticmethod
    def step_arrays(batch):
        """Which of the step's rows go to which attention kernel.

        Requests that bring at most ``ROW_KERNEL_MAX_Q`` tokens are handled row by row (``rows``;
        keys split over blocks); longer portions in tiles of consecutive queries, as many as the
        general tile kernel takes (``tiles``: first flat row and number of rows each), and the
        same portions in the larger tiles of the matrix-core kernel (``big_tiles``, the tile with
        the most keys first).  ``all_tiles`` covers every row with tiles, for head sizes the row kernels do
        not take.  ``max_row_context``: the most keys that a row of ``rows`` sees, which decides
        how its keys are split; in a step that is recorded, the length it is planned for.
        ``rows_are_requests``: 1 if every request brings one token, so that item ``i`` of ``rows``
        is row ``i`` of request ``i`` (the decode kernel then need not look either up)."""
        TILE_Q, BIG_TILE_Q = kernels.attn_tile_sizes()
        tiles, rows, all_tiles, big = [], [], [], []
        longest = 0
        for q0, n, length in zip(batch.q_starts, batch.q_lens, batch.context_lens):
            for s in range(0, n, TILE_Q):
                all_tiles += (q0 + s, min(TILE_Q, n - s))
            if n <= ROW_KERNEL_MAX_Q:
                rows += range(q0, q0 + n)
                longest = max(longest, length + n)
            else:
                for s in range(0, n, TILE_Q):
                    tiles += (q0 + s, min(TILE_Q, n - s))
                for s in range(0, n, BIG_TILE_Q):
                    m = min(BIG_TILE_Q, n - s)
                    big.append((length + s + m, q0 + s, m))
        if batch.static and rows:
            longest = batch.max_positions  # how keys are split must not depend on lengths
        big.sort(reverse=True)  # tiles with the most keys start first
        return {"tiles": tiles, "rows": rows, "all_tiles": all_tiles,
                "big_tiles": [v for _, r0, m in big for v in (r0, m)], "max_row_context": longest,
                "rows_are_requests": int(all(n == 1 for n in batch.q_lens))}

    @staticmethod
    def length_class(longest):
        """``(class, length to plan for)`` of a recorded decode step whose longest request sees
        ``longest`` keys.  Class 0 is every length below the one from which the decode kernel may
        split a row's keys over blocks, class 1 up to twice that, class 2 up to four times, and a
        step is planned for the longest of its class.  (Planned for the model's positions, a step
        of requests that are nowhere near that long would launch the blocks of splits that no row
        takes and leave fewer CUs to read weights ahead.)"""
        base = kernels.rows_split_from()
        if longest < base:
            return 0, base - 1
        c = (longest // base).bit_length()
        return c, base * (1 << c) - 1

    # -- the native twin ---------------------------------------------------------

    def make_native(self):
        L = native.lib()
        base = native.array_ids(self.step_arrays_key, self.step_array_names)
        qkv_w, out_w = kernels.weight_struct(self.qkv_w), kernels.weight_struct(self.out_w)
        pos = self.position.native() if self.position is not None else None
        return native.made(L.eng_make_attention(
            self.width, self.n_heads, self.n_kv_heads, self.head_dim, self.scale, self.window,
            ctypes.byref(qkv_w), native.ptr(self.qkv_b), ctypes.byref(out_w), native.ptr(self.out_b), pos, base),
            "attention")

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        """Fused q/k/v projection (keys and values go to their pages from its epilogue, or after
        the position hook has rotated them), attention through the block table, output projection
        added into ``residual``: done by the native twin."""
        v, r = value_of(x), native.mat(residual)
        with ctx.enter():
            rc = native.lib().eng_mixer_forward(self.native(), ctypes.byref(ctx.c), ctypes.byref(v),
                                                ctypes.byref(r), cache.slot, int(bool(writes_cache)))
        native.check(rc, "attention")


register_mixer("attention", CausalSelfAttention)
