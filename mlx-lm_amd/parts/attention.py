"""Causal self-attention over the paged cache."""

from ..config.plan import CacheNeed
from ..ops import kernels
from .base import POSITION_ENCODINGS, Mixer, TensorSpec, build_part, register_mixer


READ_AHEAD_BYTES_PER_CU = 160 * 1024  # what an idle CU reads while decode attention runs (some 5 us)


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

    def forward(self, ctx, x, residual, cache, writes_cache=True):
        T = x.shape[0]
        qkv = ctx.scratch((T, self.q_width + 2 * self.kv_width), ctx.dtype)
        q = qkv[:, : self.q_width]
        if self.position is None:
            # keys and values go to their pages from the projection's epilogue
            scatter = kernels.KVScatter(cache.kv, cache.block_table, ctx.token_req, ctx.positions,
                                        self.q_width) if writes_cache else None
            kernels.linear(qkv, x, self.qkv_w, self.qkv_b, scatter=scatter)
        else:
            kernels.linear(qkv, x, self.qkv_w, self.qkv_b)
            k = qkv[:, self.q_width : self.q_width + self.kv_width]
            v = qkv[:, self.q_width + self.kv_width :]
            self.position.rotate(ctx, q, k)
            if writes_cache:
                kernels.kv_write(k, v, cache.kv, cache.block_table, ctx.token_req, ctx.positions)
        out = ctx.scratch((T, self.q_width), ctx.dtype)
        self.attend(ctx, out, q, cache)
        kernels.linear(residual, out, self.out_w, self.out_b, accumulate=True, pending=ctx.pending)

    def attend(self, ctx, out, q, cache):
        plan = ctx.attention_plan
        args = (cache.kv, cache.block_table, ctx.token_req, ctx.positions)
        if self.head_dim > kernels.ATTN_ROW_MAX_HEAD_DIM:
            kernels.attn_tile(out, q, *args, plan.all_tiles, plan.n_all_tiles, self.n_heads,
                              self.scale, self.window)
            return
        if plan.n_tiles:
            if kernels.attn_prefill_takes(q.dtype, cache.kv):
                kernels.attn_prefill(out, q, *args, plan.big_tiles, plan.n_big_tiles, self.n_heads,
                                     self.scale, self.window)
            else:
                kernels.attn_tile(out, q, *args, plan.tiles, plan.n_tiles, self.n_heads, self.scale,
                                  self.window)
        if plan.n_rows:
            fast = kernels.attn_decode_takes(q.dtype, cache.kv)
            if fast:
                n_splits, n_waves = plan.row_work(self.n_heads, self.window)
            else:
                n_splits, n_waves = plan.row_splits(self.n_heads, self.window), 4
            part_o = part_ml = None
            if n_splits > 1:
                n = plan.n_rows * self.n_heads * n_splits
                part_o = ctx.scratch((n * self.head_dim,), "float32")
                part_ml = ctx.scratch((n * 2,), "float32")
            if fast:
                # CUs without a row read the weights that come after this mixer's own (the block
                # says which), as many chunks as they manage while the rows' blocks run; where fewer
                # than half the CUs are idle the reading slows the rows' blocks by more than it gains
                ahead, chunks = getattr(ctx, "read_ahead", None), 0
                idle = 256 - plan.n_rows * self.n_heads * n_splits
                if (ahead is not None and idle >= 128 and plan.n_tiles == 0 and plan.n_rows == q.shape[0]
                        and kernels.read_ahead_pays(ahead, plan.n_rows, with_norm=True)):
                    chunks = idle * READ_AHEAD_BYTES_PER_CU // ahead.chunk_bytes
                else:
                    ahead = None
                kernels.attn_decode(out, q, *args, plan.rows, plan.n_rows, self.n_heads, self.scale,
                                    self.window, n_splits, part_o, part_ml, n_waves, ahead=ahead,
                                    ahead_chunks=chunks)
            else:
                kernels.attn_row(out, q, *args, plan.rows, plan.n_rows, self.n_heads, self.scale,
                                 self.window, n_splits, part_o, part_ml)


register_mixer("attention", CausalSelfAttention)
