"""Steps recorded once as a HIP graph and replayed.

A step in which every request brings exactly one token and wants its logits
has the same launches every time: only the contents of the integer arrays
(token ids, positions, block tables, state slots) change.  Such a step is run
once eagerly, then captured with its host-to-device copy into a graph; later
steps of the same batch size fill the pinned host array and replay.  This
takes the place of the reference's one-step-ahead ``mx.async_eval`` pipelining
(mlx_lm/generate.py:446-451,1449-1456) as the cure for launch latency.

Any other step has the same launches as an earlier one of the same shape
(tokens and wanted places per request): a scheduler that cuts prompts into
portions of one size brings the same shapes again and again.  ``StepGraph``
records such a step; its integer arrays are built as for an eager step, but
into a device buffer of the graph's own.
"""

import contextlib
import gc
import weakref

import numpy as np
import torch

from .context import AttentionPlan, StepContext


def _pad4(n):
    return (n + 3) // 4 * 4


@contextlib.contextmanager
def _recording(graph):
    """``torch.cuda.graph(graph)`` with the cyclic garbage collector switched off.

    The collector may run at any allocation.  If it then frees a recorded graph
    that is garbage (an engine that was dropped), that graph is destroyed
    inside this capture, which HIP refuses; the error is raised in a
    destructor and ends the process.  (``torch.cuda.graph`` collects once
    before the capture begins; this keeps it from happening again within.)
    """
    was_enabled = gc.isenabled()
    gc.disable()
    try:
        with torch.cuda.graph(graph):
            yield
    finally:
        if was_enabled:
            gc.enable()


class DecodeGraph:
    """The recorded decode step for one batch size."""

    def __init__(self, engine, batch):
        # (a weak reference: the engine owns its graphs, and without a cycle they are freed
        # the moment the engine is dropped, not whenever the collector next runs)
        self.engine, self.batch = weakref.proxy(engine), batch
        cm = engine.cache
        B = batch
        self.max_blocks = cm.blocks_for(engine.decoder.max_positions)
        sizes = [B] * 6 + [2 * B] + [B * self.max_blocks] * len(cm.groups) + [B]  # last: fed rows
        self.fed_piece = len(sizes) - 1
        self.offsets, total = [], 0
        for s in sizes:
            self.offsets.append(total)
            total += _pad4(s)
        self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
        self.host_np = self.host.numpy()
        self.dev = torch.zeros(total, dtype=torch.int32, device=engine.device)
        ar = np.arange(B, dtype=np.int32)
        for i in (2, 3, 5):  # token_req, wanted rows, attention rows: row r is request r
            self.host_np[self.offsets[i] : self.offsets[i] + B] = ar
        tiles = np.stack([ar, np.ones(B, dtype=np.int32)], 1).reshape(-1)
        self.host_np[self.offsets[6] : self.offsets[6] + 2 * B] = tiles
        self._row_keys = [[None] * B for _ in cm.groups]
        self.graph = None
        self.logits = None
        self._keep = None  # buffers the recorded launches point into
        self._copied = None

    def _piece(self, i, n):
        return self.dev[self.offsets[i] : self.offsets[i] + n]

    def _context(self):
        eng, B = self.engine, self.batch
        ctx = StepContext(eng)
        ctx.n_tokens = ctx.n_requests = ctx.n_wanted = B
        ctx.wants_every_row = True
        ctx.token_ids, ctx.positions, ctx.token_req = self._piece(0, B), self._piece(1, B), self._piece(2, B)
        ctx.wanted_rows, ctx.slot_ids = self._piece(3, B), self._piece(4, B)
        plan = AttentionPlan()
        plan.rows, plan.n_rows = self._piece(5, B), B
        plan.all_tiles, plan.n_all_tiles = self._piece(6, 2 * B), B
        plan.tiles, plan.n_tiles = self._piece(6, 0), 0
        plan.max_row_context = eng.decoder.max_positions
        ctx.attention_plan = plan
        for gi in range(len(eng.cache.groups)):
            ctx.block_tables.append(self._piece(7 + gi, B * self.max_blocks).view(B, self.max_blocks))
        return ctx

    def _feed(self, ctx):
        """Tokens fed on the device replace the placeholders (a row of -1s changes nothing)."""
        from ..ops import kernels

        kernels.feed_tokens(ctx.token_ids, self.engine.fed_src, self._piece(self.fed_piece, self.batch),
                            self.engine.decoder.vocab_size)

    def _fill(self, entries):
        cm = self.engine.cache
        if self._copied is not None:
            self._copied.synchronize()  # the last replay's copy has read the host array
        h, off, B = self.host_np, self.offsets, self.batch
        for r, e in enumerate(entries):
            rc = cm.requests[e.request_id]
            h[off[0] + r] = int(e.tokens[0])
            h[off[self.fed_piece] + r] = e.fed_row
            h[off[1] + r] = rc.length
            h[off[4] + r] = rc.state_slot
            for gi in range(len(cm.groups)):
                blocks = rc.blocks[gi]
                key = (rc.serial, rc.version)  # (every edit of a table counts its version up)
                if self._row_keys[gi][r] != key:
                    base = off[7 + gi] + r * self.max_blocks
                    # pages a window has let go (-1) are never read; page 0 keeps the entry valid
                    h[base : base + len(blocks)] = [p if p >= 0 else 0 for p in blocks]
                    self._row_keys[gi][r] = key

    def run(self, entries):
        eng = self.engine
        self._fill(entries)
        if self.graph is None:
            ctx = self._context()
            # once eagerly: libraries load, scratch memory grows to what the step needs
            self.dev.copy_(self.host, non_blocking=True)
            self._feed(ctx)
            eng.scratch.reset()
            eng.decoder.forward(ctx)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            eng.scratch.frozen = True
            try:
                with _recording(graph):
                    self.dev.copy_(self.host, non_blocking=True)
                    self._feed(ctx)
                    eng.scratch.reset()
                    self.logits = eng.decoder.forward(ctx)
            finally:
                eng.scratch.frozen = False
            self.graph = graph
            self._keep = (eng.scratch.buffer, eng._logits, eng.fed_src)
            self._copied = torch.cuda.Event()
            # The step has run (eagerly, above) and recording runs nothing: replaying now would run
            # it a second time, and a mixer that keeps state would take the step's tokens twice.
            self._copied.record()
            return self.logits
        self.graph.replay()
        self._copied.record()
        return self.logits


class StepGraph:
    """A recorded step of one shape (tokens per request, number of wanted places)."""

    def __init__(self, engine):
        self.engine = weakref.proxy(engine)
        self.dev = None  # the step's integer arrays, at the same offsets every time
        self.graph = None
        self.logits = None
        self.failed = False
        self.error = None  # why recording failed, if it did
        self._keep = None

    def run(self, entries):
        eng = self.engine
        ctx = eng._build_context(entries, static=self)
        if self.graph is None:
            # once eagerly with this context (its block tables are wider, its keys may be split
            # further than in the eager steps before): scratch memory grows to what it needs
            eng.scratch.reset()
            eng.decoder.forward(ctx)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            eng.scratch.frozen = True
            try:
                with _recording(graph):
                    eng.scratch.reset()
                    self.logits = eng.decoder.forward(ctx)
            except Exception as e:
                self.failed = True  # this shape stays eager (an error of the step itself comes again below)
                self.error = e
            finally:
                eng.scratch.frozen = False
            if self.failed:
                eng.scratch.reset()
                return eng.decoder.forward(ctx)
            self.graph = graph
            self._keep = (eng.scratch.buffer, eng._logits)
            return self.logits  # (the eager run above was the step; a replay would run it again)
        self.graph.replay()
        return self.logits
