"""One packer for every kind of step: the batch's integer arrays, laid out in one buffer.

A step's parts read the batch from int32 arrays on the device: the token ids, positions and
request rows of the flat batch, the wanted rows, the state slots, one block table per cache
group, and whatever arrays the model's parts declared through ``step_arrays`` (the attention
part's work lists, for one).  ``pack`` writes them all into one pinned host buffer, pieces
starting on 16-byte boundaries, for one copy to the device.  An eager step, a recorded step and
a replay are packed by this same function; they differ in where the buffer lives
(``EagerStore``: buffers taken in turn; ``StaticStore``: a recorded step's own, at offsets that
depend on the step's shape only).
"""

import numpy as np
import torch

from .context import HostBatch, StepContext


def _pad4(n):
    return (n + 3) // 4 * 4


class EagerStore:
    """Pinned host buffers taken in turn, and one device buffer that every eager step reuses.

    A host buffer is written again only after the copy that read it has finished; the device
    buffer is safe because steps follow each other on one stream.
    """

    static = False

    def __init__(self, device, depth=4):
        self.device = device
        self.bufs = [None] * depth
        self.events = [None] * depth
        self.i = 0
        self.dev = None

    def begin(self, total):
        self.i = (self.i + 1) % len(self.bufs)
        if self.events[self.i] is not None:
            self.events[self.i].synchronize()
        b = self.bufs[self.i]
        if b is None or b.numel() < total:
            b = self.bufs[self.i] = torch.empty(max(total, 4096), dtype=torch.int32, pin_memory=True)
        if self.dev is None or self.dev.numel() < total:
            self.dev = torch.empty(max(total, 4096), dtype=torch.int32, device=self.device)
        self.total = total
        return b.numpy()

    def table_rows(self, group, n_requests):
        return None  # every row is written every step

    def send(self):
        """Queue the copy to the device."""
        self.dev[: self.total].copy_(self.bufs[self.i][: self.total], non_blocking=True)
        ev = self.events[self.i] or torch.cuda.Event()
        ev.record()
        self.events[self.i] = ev


class StaticStore:
    """A recorded step's own buffers: the same addresses and offsets at every replay.

    A request's row of a block table is written again only when the table was edited since
    (``RequestCache.version``) or the row is another request's now.
    """

    static = True

    def __init__(self, device, plan_positions=None):
        self.device = device
        self.plan_positions = plan_positions  # the length the step is planned for (None: the model's positions)
        self.host = self.host_np = self.dev = None
        self.total = None
        self.copied = None  # recorded after the copy that reads the host buffer was queued
        self._row_keys = {}

    def begin(self, total):
        if self.host is None:
            self.host = torch.zeros(total, dtype=torch.int32, pin_memory=True)
            self.host_np = self.host.numpy()
            self.dev = torch.zeros(total, dtype=torch.int32, device=self.device)
            self.total = total
        if total != self.total:
            raise RuntimeError("a recorded step's arrays changed size")
        if self.copied is not None:
            self.copied.synchronize()  # the last replay's copy has read the host array
        return self.host_np

    def table_rows(self, group, n_requests):
        keys = self._row_keys.get(group)
        if keys is None or len(keys) != n_requests:
            keys = self._row_keys[group] = [None] * n_requests
        return keys

    def send(self):
        self.dev.copy_(self.host, non_blocking=True)

    def sent(self):
        if self.copied is None:
            self.copied = torch.cuda.Event()
        self.copied.record()


def pack(engine, entries, store):
    """Lay out the arrays of the step ``entries`` in ``store`` and return its ``StepContext``.

    Nothing is copied or launched here; ``store.send()`` queues the copy.
    """
    cm = engine.cache
    dec = engine.decoder
    R = len(entries)
    reqs = [cm.requests[e.request_id] for e in entries]
    q_lens = [len(e.tokens) for e in entries]
    context_lens = [rc.length for rc in reqs]
    state_slots = [rc.state_slot for rc in reqs]
    T = sum(q_lens)
    q_starts, s = [], 0
    for n in q_lens:
        q_starts.append(s)
        s += n
    static = store.static
    batch = HostBatch(q_starts, q_lens, context_lens, state_slots, static,
                      getattr(store, "plan_positions", None) or dec.max_positions)

    if T == R:  # one token a request: no repeats to spell out
        token_ids = [e.tokens[0] for e in entries]
        positions = context_lens
        token_req = np.arange(R, dtype=np.int32)
        fed_index = [e.fed_row if e.fed_row >= 0 else -1 for e in entries]
    else:
        lens = np.asarray(q_lens, dtype=np.int64)
        token_ids = np.concatenate([np.asarray(e.tokens, dtype=np.int32) for e in entries])
        token_req = np.repeat(np.arange(R, dtype=np.int32), lens)
        starts = np.repeat(np.asarray(q_starts, dtype=np.int64), lens)
        positions = (np.arange(T, dtype=np.int64) - starts
                     + np.repeat(np.asarray(context_lens, dtype=np.int64), lens)).astype(np.int32)
        fed_index = np.repeat(np.asarray([e.fed_row if e.fed_row >= 0 else -1 for e in entries],
                                         dtype=np.int32), lens)
    wanted = [qs + w for e, qs in zip(entries, q_starts) for w in e.want]
    n_wanted = len(wanted)
    every = n_wanted == T and wanted == list(range(T))

    # name -> (values or scalar); the standard arrays first, then the parts' own, then the tables
    pieces = [("token_ids", token_ids, T), ("positions", positions, T), ("token_req", token_req, T),
              ("wanted_rows", wanted, n_wanted), ("slot_ids", state_slots, R), ("fed_index", fed_index, T)]
    part_arrays = []  # (array id, name, values or None, count or scalar)
    for base, key, names, provider in engine.array_providers:
        got = provider(batch)
        for i, name in enumerate(names):
            v, name = got[name], f"{key}.{name}"
            if isinstance(v, (int, np.integer)):
                part_arrays.append((base + i, name, None, int(v)))
            else:
                part_arrays.append((base + i, name, v, len(v)))
                pieces.append((name, v, len(v)))
    widths = []
    for gi in range(len(cm.groups)):
        width = cm.blocks_for(dec.max_positions) if static else max(1, max(len(rc.blocks[gi]) for rc in reqs))
        widths.append(width)
        pieces.append((("table", gi), None, R * width))

    offsets, total = {}, 0
    for name, _, n in pieces:
        offsets[name] = total
        total += _pad4(n)
    host = store.begin(total)
    for name, v, n in pieces:
        if v is not None and n:
            host[offsets[name] : offsets[name] + n] = v
    for gi, width in enumerate(widths):
        off = offsets[("table", gi)]
        keys = store.table_rows(gi, R)
        for r, rc in enumerate(reqs):
            blocks = rc.blocks[gi]
            if keys is not None:
                key = (rc.serial, rc.version)  # (every edit of a table counts its version up)
                if keys[r] == key:
                    continue
                keys[r] = key
            base = off + r * width
            host[base : base + len(blocks)] = blocks
            if not static:
                host[base + len(blocks) : base + width] = -1

    ctx = StepContext(engine)
    ctx.q_starts, ctx.q_lens, ctx.context_lens, ctx.state_slots = q_starts, q_lens, context_lens, state_slots
    ctx.n_tokens, ctx.n_requests, ctx.n_wanted, ctx.wants_every_row = T, R, n_wanted, every
    ctx.any_fed = any(e.fed_row >= 0 for e in entries)
    dev = store.dev
    ctx.bind(dev, offsets, {"token_ids": T, "positions": T, "token_req": T, "wanted_rows": n_wanted,
                            "slot_ids": R, "fed_index": T}, part_arrays, widths)
    return ctx
