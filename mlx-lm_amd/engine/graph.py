"""Steps recorded once as a HIP graph and replayed.

A step has the same launches as an earlier one of the same shape (tokens and wanted places per
request): only the contents of the integer arrays (token ids, positions, block tables, state
slots, work lists) change.  Such a step is run once eagerly, then captured with its
host-to-device copy into a graph; later steps of the same shape fill the graph's own pinned host
array and replay.  Decode steps (one token a request, all logits wanted) are recorded per batch
size at their first sighting; a scheduler that cuts prompts into portions of one size brings
other shapes again and again, and those are recorded where the engine is asked to.  This takes
the place of the reference's one-step-ahead ``mx.async_eval`` pipelining
(mlx_lm/generate.py:446-451,1449-1456) as the cure for launch latency.

The arrays are packed by the same function as an eager step's (``pack.pack``), into a
``StaticStore``: block tables of full width, and nothing about the launches may depend on the
requests' lengths.
"""

import contextlib
import gc
import weakref

import torch

from .pack import StaticStore, pack


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


class StepGraph:
    """A recorded step of one shape (tokens per request, number of wanted places)."""

    def __init__(self, engine, plan_positions=None):
        # (a weak reference: the engine owns its graphs, and without a cycle they are freed
        # the moment the engine is dropped, not whenever the collector next runs)
        self.engine = weakref.proxy(engine)
        self.store = StaticStore(engine.device, plan_positions)
        self.graph = None
        self.logits = None
        self.failed = False
        self.error = None  # why recording failed, if it did
        self._keep = None  # buffers the recorded launches point into

    def _launches(self, ctx):
        eng = self.engine
        self.store.send()
        if 1 in ctx.q_lens:
            # tokens fed on the device replace the placeholders (a row of -1s changes nothing)
            from ..ops import kernels

            kernels.feed_tokens(ctx.token_ids, eng.fed_src, ctx.fed_index, eng.decoder.vocab_size)
        eng.scratch.reset()
        return eng.decoder.forward(ctx)

    def run(self, entries):
        eng = self.engine
        ctx = pack(eng, entries, self.store)
        if self.graph is not None:
            self.graph.replay()
            self.store.sent()
            return self.logits
        # Once eagerly with this context (its block tables are wider, its keys may be split
        # further than in an eager step's): libraries load, scratch memory grows to what the
        # step needs.  This run is the step: recording runs nothing, and a replay on top would
        # run the step a second time (a mixer that keeps state would take its tokens twice).
        logits = self._launches(ctx)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        eng.scratch.frozen = True
        try:
            with _recording(graph):
                self.logits = self._launches(ctx)
        except Exception as e:
            self.failed = True  # this shape stays eager
            self.error = e
        finally:
            eng.scratch.frozen = False
        if not self.failed:
            self.graph = graph
            self._keep = (eng.scratch.buffer, eng._logits, eng.fed_src)
        self.store.sent()
        return logits
