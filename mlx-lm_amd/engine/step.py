"""The step function: one batch of (request, its next tokens) through the model."""

from collections import OrderedDict
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

from ..cache import CacheManager
from ..weights.loader import resolve_dtype
from ..ops import native
from .context import Scratch
from .pack import EagerStore, pack


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
        if len(self.cache.groups) > native.MAX_GROUPS:
            raise ValueError(
                f"the model's cache slots fall into {len(self.cache.groups)} groups of different needs; "
                f"a step carries at most {native.MAX_GROUPS} block tables (ENG_MAX_GROUPS in csrc/engine.h)")
        self.scratch = Scratch(self.device)
        self._eager = EagerStore(self.device)
        self._logits = None
        self.steps = 0
        # what the native parts need of the device and the cache, made once
        from ..ops import kernels

        native.lib()
        self.n_compute_units = kernels.n_compute_units()
        self.split_ws = kernels.split_workspace(self.device)
        self.stats = native.EngStats()
        self.slot_table = self._slot_table()
        self.array_providers = self.decoder.array_providers()
        # sampled tokens that go into the next step without passing through the host
        self.fed_src = torch.zeros(max(64, max_requests), dtype=torch.int32, device=self.device)
        # decode steps are recorded as graphs where every part launches kernels only
        self.use_graphs = use_graphs and all(getattr(p, "graph_safe", False) for p in self.decoder.parts())
        self._graphs = {}
        self._length_classers = None  # the parts that put recorded decode steps into classes of length
        # Other steps whose shape keeps coming back (portions of prompts of the scheduler's size, with
        # or without decoding requests beside them) are recorded too, if asked for.
        self.record_prompt_steps = bool(record_prompt_steps) and self.use_graphs
        self._step_graphs = OrderedDict()
        self._shape_seen = {}

    def _slot_table(self):
        """One ``EngSlot`` per cache slot: where its pages lie and which block table is its group's."""
        cm = self.cache
        n = max([-1, *cm.slot_group, *cm.state_needs]) + 1
        n = max(n, len(self.decoder.cache_needs()))
        table = (native.EngSlot * max(n, 1))()
        for slot in range(n):
            s = table[slot]
            s.group = -1
            if slot in cm.slot_group:
                g, _ = cm.slot_group[slot]
                k, v = cm.kv(slot)
                need = cm.groups[g].need
                s.k, s.v, s.page_stride, s.v_page_stride = k.data_ptr(), v.data_ptr(), k.stride(0), v.stride(0)
                s.n_kv_heads, s.head_dim, s.page_size = need.n_kv_heads, need.head_dim, cm.page_size
                s.v_head_dim = need.value_dim
                s.dtype, s.group = native.DT[k.dtype], g
            elif slot in cm.state_needs:
                # per-request state: the tensor, and how many elements a request's row holds
                state = cm.state(slot)
                s.k, s.page_stride = state.data_ptr(), state.stride(0)
                s.dtype, s.group = native.DT.get(state.dtype, -1), -2
        return table

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

    def detach_request(self, request_id):
        """End a request but keep what it computed (its pages stay held): ``KeptPages`` that
        ``attach_request`` makes a request of again and ``drop_kept`` gives back."""
        return self.cache.detach(request_id)

    def attach_request(self, request_id, kept):
        return self.cache.attach(request_id, kept)

    def drop_kept(self, kept):
        self.cache.drop(kept)

    def read_kept(self, kept):
        """``KeptPages`` as tensors of their own (``CacheManager.read_kept``)."""
        return self.cache.read_kept(kept)

    def write_kept(self, length, per_slot, state):
        """Pages of this engine's pool that hold the given keys, values and state rows."""
        return self.cache.write_kept(length, per_slot, state)

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

        try:
            graph = self._recorded_step(entries) if self.use_graphs else None
            if graph is not None:
                logits = graph.run(entries)
            else:
                ctx = self._build_context(entries)
                self.scratch.reset()
                logits = self.decoder.forward(ctx)
        except Exception:
            # a step that raised has stored nothing that counts: its pages go back as above
            for rid, mark in marks:
                cm.rollback(rid, mark)
            raise
        for e in entries:
            cm.commit(e.request_id, len(e.tokens))
        self.steps += 1
        return logits

    RECORD_AFTER = 2  # sightings of a shape before its step is recorded
    MAX_RECORDED = 24

    def _recorded_step(self, entries):
        """The recorded step for this batch's shape, if it has one (or is due one).

        A step in which every request brings one token and wants its logits (a decode step) is
        recorded at its first sighting; steps of other shapes after ``RECORD_AFTER`` sightings,
        and only where ``record_prompt_steps`` asks for it."""
        q_lens = tuple(len(e.tokens) for e in entries)
        n_wanted = sum(len(e.want) for e in entries)
        every = n_wanted == sum(q_lens) and all(list(e.want) == list(range(len(e.tokens))) for e in entries)
        decode = every and n_wanted == len(entries)
        if decode:
            # one recorded step for each number of requests and class of length: a step is planned
            # for the longest request of its class, not for the model's positions
            longest = max(self.cache.requests[e.request_id].length for e in entries) + 1
            classes, plan_positions = self._length_class(longest)
            key = (len(entries), classes)
            graph = self._graphs.get(key)
            if graph is None:
                from .graph import StepGraph

                graph = self._graphs[key] = StepGraph(self, plan_positions)
            return None if graph.failed else graph
        if not self.record_prompt_steps:
            return None
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

    def _length_class(self, longest):
        """``(classes, length to plan for)`` of a recorded decode step whose longest request holds
        ``longest`` tokens: what the parts that have a ``length_class`` say (one answer a kind of
        part), and the largest of their lengths, at most the model's positions."""
        if self._length_classers is None:
            kinds = {}
            for p in self.decoder.parts():
                if hasattr(p, "length_class"):
                    kinds.setdefault(type(p), p)
            self._length_classers = list(kinds.values())
        classes, plan = [], 0
        for p in self._length_classers:
            c, n = p.length_class(longest)
            classes.append(c)
            plan = max(plan, n)
        P = self.decoder.max_positions
        return tuple(classes), (min(plan, P) if classes else P)

    def _build_context(self, entries):
        """The context of an eager step: its arrays packed and on their way to the device, tokens
        that are still on the device fed into their places."""
        ctx = pack(self, entries, self._eager)
        self._eager.send()
        self.feed(ctx)
        return ctx

    def feed(self, ctx):
        """Tokens fed on the device replace the placeholders of their entries."""
        if ctx.any_fed:
            from ..ops import kernels

            kernels.feed_tokens(ctx.token_ids, self.fed_src, ctx.fed_index, self.decoder.vocab_size)
