"""The step function: one batch of (request, its next tokens) through the model."""

from collections import OrderedDict
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

from ..cache import CacheManager
from ..weights.loader import resolve_dtype
from .context import BIG_TILE_Q, ROW_KERNEL_MAX_Q, TILE_Q, AttentionPlan, Scratch, StepContext


@dataclass
class StepEntry:
    """A request's share of a step: its next tokens and the places, among
    these tokens, whose logits are wanted."""

    request_id: object
    tokens: Sequence[int]
    want: Sequence[int] = ()
    # Row of the step's ``fed`` tokens (sampled tokens still on the device) that is
    # this request's one token; ``tokens`` then holds a placeholder.  -1: ``tokens`` are the tokens.
    fed_row: int = -1


class _HostRing:
    """Pinned host buffers for the step's integer arrays, reused in turn.

    A buffer is written again only after the copy that read it has finished.
    """

    def __init__(self, n=4):
        self.bufs = [None] * n
        self.events = [None] * n
        self.i = 0

    def get(self, n_ints):
        self.i = (self.i + 1) % len(self.bufs)
        if self.events[self.i] is not None:
            self.events[self.i].synchronize()
        b = self.bufs[self.i]
        if b is None or b.numel() < n_ints:
            b = torch.empty(max(n_ints, 4096), dtype=torch.int32, pin_memory=True)
            self.bufs[self.i] = b
        return b

    def current(self):
        return self.bufs[self.i]

    def mark(self):
        ev = self.events[self.i] or torch.cuda.Event()
        ev.record()
        self.events[self.i] = ev


class Engine:
    """A model, its cache and the step function over them.

    ``step(entries)`` runs exactly the tokens it is given as one flat batch --
    portions of prompts beside single decoded tokens, cut anywhere -- against
    what earlier steps left in the cache, and returns float32 logits at the
    wanted places.  The reference's forward takes a rectangle of tokens and
    returns logits everywhere (mlx_lm/models/gpt2.py:161-168); callers there
    slice or drop them (mlx_lm/generate.py:398,424-431,1244,1415).
    """

    def __init__(self, model, dtype="bfloat16", device="cuda:0", page_size=16, n_pages=None,
                 max_tokens=None, max_requests=64, use_graphs=True, record_prompt_steps=False):
        if not torch.cuda.is_available():
            raise RuntimeError("the engine needs a GPU: torch.cuda.is_available() is false")
        self.model = model
        self.decoder = model.decoder
        self.dtype = resolve_dtype(dtype)
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        if n_pages is None:
            if max_tokens is None:
                raise ValueError("give the cache size as n_pages or max_tokens")
            n_pages = (max_tokens + page_size - 1) // page_size
        self.cache = CacheManager(self.decoder.cache_needs(), page_size, n_pages, max_requests,
                                  dtype=self.dtype, device=self.device)
        self.scratch = Scratch(self.device)
        self._ring = _HostRing()
        self._meta_dev = None
        self._logits = None
        self.steps = 0
        # sampled tokens that go into the next step without passing through the host
        self.fed_src = torch.zeros(max(64, max_requests), dtype=torch.int32, device=self.device)
        # decode steps are recorded as graphs where every part launches kernels only
        self.use_graphs = use_graphs and all(getattr(p, "graph_safe", False) for p in self.decoder.parts())
        self._graphs = {}
        # Other steps whose shape keeps coming back (portions of prompts of the scheduler's size, with
        # or without decoding requests beside them) are recorded too, if asked for.
        self.record_prompt_steps = bool(record_prompt_steps) and self.use_graphs
        self._step_graphs = OrderedDict()
        self._shape_seen = {}

    # -- buffers ---------------------------------------------------------------

    def logits_buffer(self, n_rows, vocab):
        if self._logits is None or self._logits.shape[0] < n_rows or self._logits.shape[1] != vocab:
            self._logits = torch.empty((max(n_rows, 8), vocab), dtype=torch.float32, device=self.device)
        return self._logits[:n_rows]

    # -- requests --------------------------------------------------------------

    def add_request(self, request_id):
        return self.cache.add(request_id)

    def end_request(self, request_id):
        self.cache.release(request_id)

    def has_request(self, request_id):
        return request_id in self.cache.requests

    def context_len(self, request_id):
        return self.cache.requests[request_id].length

    def truncate(self, request_id, new_length):
        """Forget a request's tokens from ``new_length`` on; the next step goes on from there.

        ``trim_prompt_cache`` of the reference (mlx_lm/models/cache.py:91-107,378-381) counts
        the tokens to drop; see ``trim``.  Pages beyond the new end are given back at once.  A
        mixer that keeps state of fixed size cannot go back (mlx_lm/models/cache.py:146-147):
        a model with one refuses.
        """
        if self.cache.state_needs:
            raise ValueError("a model whose mixers keep per-request state cannot be trimmed")
        return self.cache.truncate(request_id, new_length).length

    def trim(self, request_id, n_tokens):
        """Drop the last ``n_tokens`` tokens of a request (at most all); returns how many went."""
        n = max(0, min(int(n_tokens), self.context_len(request_id)))
        self.truncate(request_id, self.context_len(request_id) - n)
        return n

    # -- the step --------------------------------------------------------------

    def _check(self, entries):
        seen = set()
        V, P = self.decoder.vocab_size, self.decoder.max_positions
        for e in entries:
            if e.request_id in seen:
                raise ValueError(f"request {e.request_id!r} occurs twice in one step")
            seen.add(e.request_id)
            if e.request_id not in self.cache.requests:
                raise KeyError(f"request {e.request_id!r} is not live")
            n = len(e.tokens)
            if n == 0:
                raise ValueError(f"request {e.request_id!r} brings no tokens")
            if e.fed_row >= 0 and n != 1:
                raise ValueError(f"request {e.request_id!r}: a token fed on the device is one token")
            if n == 1:  # (the common case, without an array)
                t = e.tokens[0]
                if not 0 <= t < V:
                    raise ValueError(f"token id {int(t)} of request {e.request_id!r} is outside [0, {V})")
            else:
                toks = np.asarray(e.tokens, dtype=np.int64)
                if toks.ndim != 1 or int(toks.min()) < 0 or int(toks.max()) >= V:
                    bad = [int(t) for t in np.ravel(toks) if not 0 <= int(t) < V][:1]
                    raise ValueError(f"token id {bad[0] if bad else '?'} of request {e.request_id!r} is outside [0, {V})")
            length = self.cache.requests[e.request_id].length
            if length + n > P:
                raise ValueError(
                    f"request {e.request_id!r} would reach {length + n} tokens, the model "
                    f"has {P} positions"
                )
            for w in e.want:
                if not 0 <= w < n:
                    raise ValueError(f"wanted place {int(w)} of request {e.request_id!r} is outside its {n} tokens")

    def step(self, entries: List[StepEntry], fed=None):
        """Run one batch; returns float32 logits ``[n_wanted, vocab]`` (``None`` if nothing is wanted).

        ``fed``: an int32 device tensor of sampled tokens; entries with
        ``fed_row >= 0`` take their token from it on the device, so the step
        can be launched before the host has read those tokens.
        The returned tensor is a view of a buffer that the next step overwrites.
        """
        if not entries:
            return None
        self._check(entries)
        if any(e.fed_row >= 0 for e in entries):
            if fed is None or fed.dtype != torch.int32 or not fed.is_cuda:
                raise ValueError("entries with fed_row need the int32 device tensor `fed`")
            if fed.numel() > self.fed_src.numel() or any(e.fed_row >= fed.numel() for e in entries):
                raise ValueError(f"`fed` has {fed.numel()} tokens; at most {self.fed_src.numel()}, and every fed_row inside")
            self.fed_src[: fed.numel()].copy_(fed.reshape(-1), non_blocking=True)
        cm = self.cache
        # pages first: all or nothing for the whole step
        marks = []
        try:
            for e in entries:
                marks.append((e.request_id, cm.mark(e.request_id)))
                cm.reserve(e.request_id, len(e.tokens))
        except Exception:
            # only what this step took goes back: pages that a request held before (its whole
            # prompt's, taken at admission) stay its own
            for rid, mark in marks:
                cm.rollback(rid, mark)
            raise

        if self.use_graphs and all(len(e.tokens) == 1 and list(e.want) == [0] for e in entries):
            graph = self._graphs.get(len(entries))
            if graph is None:
                from .graph import DecodeGraph

                graph = self._graphs[len(entries)] = DecodeGraph(self, len(entries))
            logits = graph.run(entries)
        elif self.record_prompt_steps and (graph := self._recorded_step(entries)) is not None:
            logits = graph.run(entries)
        else:
            ctx = self._build_context(entries)
            self.scratch.reset()
            logits = self.decoder.forward(ctx)
        for e in entries:
            cm.commit(e.request_id, len(e.tokens))
        self.steps += 1
        return logits

    RECORD_AFTER = 2  # sightings of a shape before its step is recorded
    MAX_RECORDED = 24

    def _recorded_step(self, entries):
        """The recorded step for this batch's shape, if it has one (or is due one)."""
        q_lens = tuple(len(e.tokens) for e in entries)
        n_wanted = sum(len(e.want) for e in entries)
        every = n_wanted == sum(q_lens) and all(list(e.want) == list(range(len(e.tokens))) for e in entries)
        key = (q_lens, n_wanted, every)
        graph = self._step_graphs.get(key)
        if graph is not None:
            self._step_graphs.move_to_end(key)
            return None if graph.failed else graph
        seen = self._shape_seen.get(key, 0)
        if seen < self.RECORD_AFTER:
            if len(self._shape_seen) > 4096:
                self._shape_seen.clear()
            self._shape_seen[key] = seen + 1
            return None
        from .graph import StepGraph

        graph = self._step_graphs[key] = StepGraph(self)
        self._shape_seen.pop(key, None)
        while len(self._step_graphs) > self.MAX_RECORDED:
            self._step_graphs.popitem(last=False)
        return graph

    def _build_context(self, entries, static=None):
        """The step's context.  ``static`` (a ``StepGraph``): the integer arrays go to that graph's own
        device buffer, at offsets that depend on the step's shape only."""
        cm = self.cache
        R = len(entries)
        T = sum(len(e.tokens) for e in entries)
        ctx = StepContext(self)
        q_start = 0
        token_ids, positions, token_req, wanted, slot_ids, fed_index = [], [], [], [], [], []
        tiles, rows, all_tiles, big = [], [], [], []
        plan = AttentionPlan()
        for r, e in enumerate(entries):
            rc = cm.requests[e.request_id]
            n = len(e.tokens)
            ctx.q_starts.append(q_start)
            ctx.q_lens.append(n)
            ctx.context_lens.append(rc.length)
            token_ids.append(np.asarray(e.tokens, dtype=np.int32))
            fed_index.append(np.full(n, e.fed_row if e.fed_row >= 0 else -1, dtype=np.int32))
            positions.append(np.arange(rc.length, rc.length + n, dtype=np.int32))
            token_req.append(np.full(n, r, dtype=np.int32))
            wanted.append(q_start + np.asarray(e.want, dtype=np.int32))
            slot_ids.append(rc.state_slot)
            ctx.state_slots.append(rc.state_slot)
            for s in range(0, n, TILE_Q):
                all_tiles.extend((q_start + s, min(TILE_Q, n - s)))
            if n <= ROW_KERNEL_MAX_Q:
                rows.extend(range(q_start, q_start + n))
                plan.max_row_context = max(plan.max_row_context, rc.length + n)
            else:
                for s in range(0, n, TILE_Q):
                    tiles.extend((q_start + s, min(TILE_Q, n - s)))
                for s in range(0, n, BIG_TILE_Q):
                    big.append((rc.length + s + min(BIG_TILE_Q, n - s), q_start + s, min(BIG_TILE_Q, n - s)))
            q_start += n
        plan.n_tiles, plan.n_rows, plan.n_all_tiles = len(tiles) // 2, len(rows), len(all_tiles) // 2
        if static is not None and rows:
            plan.max_row_context = self.decoder.max_positions  # how keys are split must not depend on lengths
        big.sort(reverse=True)  # tiles with the most keys start first
        big_tiles = [v for _, r0, nr in big for v in (r0, nr)]
        plan.n_big_tiles = len(big)

        # block tables, one per group, padded to the longest of the step
        tables = []
        for gi in range(len(cm.groups)):
            width = max(1, max(len(cm.requests[e.request_id].blocks[gi]) for e in entries))
            if static is not None:
                width = cm.blocks_for(self.decoder.max_positions)
            flat = []
            for e in entries:
                b = cm.requests[e.request_id].blocks[gi]
                flat.extend(b)
                flat.extend([-1] * (width - len(b)))
            tables.append((width, flat))

        # everything in one pinned buffer and one copy; pieces start on 4-int boundaries
        token_ids, positions, token_req = (np.concatenate(x) for x in (token_ids, positions, token_req))
        wanted, fed_index = np.concatenate(wanted), np.concatenate(fed_index)
        pieces = [token_ids, positions, token_req, wanted, slot_ids, tiles, rows, all_tiles, big_tiles]
        pieces += [flat for _, flat in tables]
        pieces.append(fed_index)  # (last: the pieces before it keep their numbers)
        offsets, total = [], 0
        for p in pieces:
            offsets.append(total)
            total += (len(p) + 3) // 4 * 4
        host = self._ring.get(total).numpy()
        for off, p in zip(offsets, pieces):
            if len(p):
                host[off : off + len(p)] = p
        if static is not None:
            if static.dev is None:
                static.dev = torch.empty(total, dtype=torch.int32, device=self.device)
            if static.dev.numel() != total:
                raise RuntimeError("a recorded step's arrays changed size")
            dev = static.dev
        else:
            if self._meta_dev is None or self._meta_dev.numel() < total:
                self._meta_dev = torch.empty(max(total, 4096), dtype=torch.int32, device=self.device)
            dev = self._meta_dev
        dev[:total].copy_(self._ring.current()[:total], non_blocking=True)
        self._ring.mark()

        def piece(i, n):
            return dev[offsets[i] : offsets[i] + n]

        ctx.n_tokens, ctx.n_requests, ctx.n_wanted = T, R, len(wanted)
        ctx.wants_every_row = len(wanted) == T and bool((wanted == np.arange(T, dtype=np.int32)).all())
        ctx.token_ids, ctx.positions, ctx.token_req = piece(0, T), piece(1, T), piece(2, T)
        ctx.wanted_rows, ctx.slot_ids = piece(3, len(wanted)), piece(4, R)
        plan.tiles, plan.rows, plan.all_tiles = piece(5, len(tiles)), piece(6, len(rows)), piece(7, len(all_tiles))
        plan.big_tiles = piece(8, len(big_tiles))
        ctx.attention_plan = plan
        for gi, (width, flat) in enumerate(tables):
            ctx.block_tables.append(piece(9 + gi, len(flat)).view(R, width))
        if bool((fed_index >= 0).any()):
            from ..ops import kernels

            kernels.feed_tokens(ctx.token_ids, self.fed_src, piece(9 + len(tables), T), self.decoder.vocab_size)
        return ctx
