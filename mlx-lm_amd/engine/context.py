"""What a step's parts see: the flat batch on the device, cache views, scratch memory.

The native parts read the step from ``StepContext.c`` (an ``EngCtx`` struct); the attributes
beside it (torch views of the same arrays, host lists of where each request's tokens lie) are
for parts written in Python.
"""

import ctypes

import torch

from ..ops import native

_TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}


class Scratch:
    """A bump allocator over one device buffer, reset at every step.

    The same sequence of requests gives the same addresses, so a step's
    launches can be recorded and replayed.  The buffer grows (outside of a
    recording) when a step needs more than any step before.  Where the next
    piece starts is kept in a struct that the native parts share, so their
    pieces and those of parts written in Python follow each other.
    """

    ALIGN = 256

    def __init__(self, device, initial_bytes=1 << 20):
        self.device = device
        self.c = native.EngScratch()
        self._old = []  # outgrown buffers, kept alive until the next reset
        self._set_buffer(torch.empty(initial_bytes, dtype=torch.uint8, device=device))

    def _set_buffer(self, buffer):
        self.buffer = buffer
        self.c.base, self.c.size = buffer.data_ptr(), buffer.numel()

    @property
    def offset(self):
        return self.c.offset

    @offset.setter
    def offset(self, value):
        self.c.offset = value

    @property
    def peak(self):
        return self.c.peak

    @property
    def frozen(self):
        return bool(self.c.frozen)

    @frozen.setter
    def frozen(self, value):
        self.c.frozen = 1 if value else 0

    def reset(self):
        self.c.offset = 0
        self._old.clear()

    def grow(self, nbytes):
        """Room for ``nbytes`` in all; pieces handed out before stay valid until the next reset."""
        if nbytes <= self.buffer.numel():
            return
        if self.frozen:
            raise RuntimeError("scratch memory would have to grow while a step is being recorded")
        self._old.append(self.buffer)
        self._set_buffer(torch.empty(max(nbytes, 2 * self.buffer.numel()), dtype=torch.uint8, device=self.device))

    def take(self, shape, dtype):
        dtype = _TORCH_DTYPES.get(dtype, dtype)
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        start = (self.c.offset + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        end = start + nbytes
        if end > self.buffer.numel():
            self.grow(end)
        self.c.offset = end
        self.c.peak = max(self.c.peak, end)
        return self.buffer[start:end].view(dtype).view(*shape)

    def view(self, p, n_bytes):
        """The bytes at device address ``p`` if they lie in this allocator's memory, else ``None``."""
        for buf in [self.buffer] + self._old:
            base = buf.data_ptr()
            if base <= p and p + n_bytes <= base + buf.numel():
                return buf[p - base : p - base + n_bytes]
        return None


class _DeviceArray:
    """Memory at a device address, for ``torch.as_tensor`` (the CUDA array interface)."""

    def __init__(self, p, n_bytes):
        self.__cuda_array_interface__ = {"shape": (n_bytes,), "typestr": "|u1", "data": (p, False), "version": 2}


class CacheView:
    """One cache slot as a mixer sees it in a step: ``keys``/``values`` are the slot's pages
    (``[n_pages, n_kv_heads, page, width]`` each, of widths of their own), ``kv`` the same for the
    attention kernels here where both have one width, ``block_table`` the requests' page numbers,
    ``state`` a slot of fixed-size state."""

    __slots__ = ("kv", "keys", "values", "block_table", "state", "slot")

    def __init__(self, slot, kv=None, block_table=None, state=None, keys=None, values=None):
        self.slot, self.kv, self.block_table, self.state = slot, kv, block_table, state
        self.keys, self.values = keys, values


class HostBatch:
    """A step's batch as the host knows it, before anything is on the device: what a part's
    ``step_arrays`` gets.

    ``q_starts[r]``, ``q_lens[r]`` say where request ``r``'s tokens lie in the flat batch,
    ``context_lens[r]`` how many tokens it held before.  ``static``: the arrays are for a step
    that is recorded and replayed, so nothing about the launches (how many ways keys are split)
    may depend on the lengths; ``max_positions`` is then the length to plan for (the model's
    positions, or fewer where the parts put recorded steps into classes of length,
    ``length_class``).
    """

    __slots__ = ("q_starts", "q_lens", "context_lens", "state_slots", "n_tokens", "static", "max_positions")

    def __init__(self, q_starts, q_lens, context_lens, state_slots, static, max_positions):
        self.q_starts, self.q_lens, self.context_lens = q_starts, q_lens, context_lens
        self.state_slots, self.static, self.max_positions = state_slots, static, max_positions
        self.n_tokens = sum(q_lens)


class StepContext:
    """One step's batch, as the parts see it.

    Tokens of all requests lie in one flat list.  ``token_ids``, ``positions``
    and ``token_req`` (row of the request in the block tables) are int32
    device arrays over the tokens; ``slot_ids`` gives each request's state
    slot; ``wanted_rows`` the flat rows whose logits are asked for; ``arrays``
    holds what parts asked for through their ``step_arrays``, by name.  The host
    lists ``q_starts``/``q_lens``/``context_lens`` (tokens before this step)
    say where each request's run lies, ``state_slots`` is ``slot_ids`` on the host.
    """

    def __init__(self, engine):
        from ..ops.kernels import PendingSum

        self.engine = engine
        self.dtype = engine.dtype
        self.device = engine.device
        self._scratch = engine.scratch
        self.c = native.EngCtx()
        c = self.c
        c.dtype = native.DT[self.dtype]
        c.scratch = ctypes.pointer(engine.scratch.c)
        c.slots, c.n_slots = engine.slot_table, len(engine.slot_table)
        c.n_compute_units = engine.n_compute_units
        c.split_ws, c.split_ws_floats = engine.split_ws.data_ptr(), engine.split_ws.numel()
        c.stats = ctypes.pointer(engine.stats)
        self.n_tokens = self.n_requests = self.n_wanted = 0
        self.wants_every_row = False  # wanted_rows is 0 .. n_tokens - 1
        self.any_fed = False  # some entry's token is still on the device
        self._where = {}  # name of an array -> (offset, length) in the step's device buffer
        self._widths = []
        self._tensors = {}
        self.q_starts, self.q_lens, self.context_lens, self.state_slots = [], [], [], []
        self._views = {}
        self._kept = []  # tensors that the native side holds pointers to until the step is over
        self._meta = None  # the device buffer that holds the step's integer arrays
        # a projection's sum into the residual stream that the next norm will add
        self.pending = PendingSum(self.c.pending, self)

    # -- the step's arrays ------------------------------------------------------

    def bind(self, dev, offsets, counts, part_arrays, widths):
        """Point the native struct at the step's arrays in ``dev`` (the packer calls this)."""
        self._meta = dev
        base = dev.data_ptr()
        c = self.c
        c.n_tokens, c.n_requests, c.n_wanted = self.n_tokens, self.n_requests, self.n_wanted
        c.wants_every_row = 1 if self.wants_every_row else 0
        c.token_ids = base + 4 * offsets["token_ids"]
        c.positions = base + 4 * offsets["positions"]
        c.token_req = base + 4 * offsets["token_req"]
        c.wanted_rows = base + 4 * offsets["wanted_rows"]
        c.slot_ids = base + 4 * offsets["slot_ids"]
        where = {name: (offsets[name], n) for name, n in counts.items()}
        for aid, name, values, n in part_arrays:
            c.counts[aid] = n
            if values is not None:
                c.arrays[aid] = base + 4 * offsets[name]
                where[name] = (offsets[name], n)
            else:
                where[name] = n
        for gi, w in enumerate(widths):
            c.block_tables[gi] = base + 4 * offsets[("table", gi)]
            c.table_width[gi] = w
            where[("table", gi)] = (offsets[("table", gi)], self.n_requests * w)
        self._where, self._widths = where, list(widths)

    def array(self, name):
        """The int32 device array ``name`` of this step (a scalar comes back as an ``int``)."""
        t = self._tensors.get(name)
        if t is None:
            w = self._where[name]
            if isinstance(w, int):
                return w
            t = self._tensors[name] = self._meta[w[0] : w[0] + w[1]]
        return t

    token_ids = property(lambda self: self.array("token_ids"))
    positions = property(lambda self: self.array("positions"))
    token_req = property(lambda self: self.array("token_req"))
    wanted_rows = property(lambda self: self.array("wanted_rows"))
    slot_ids = property(lambda self: self.array("slot_ids"))
    fed_index = property(lambda self: self.array("fed_index"))

    @property
    def block_tables(self):
        """One ``[requests, blocks]`` table per cache group."""
        return [self.array(("table", gi)).view(self.n_requests, w) for gi, w in enumerate(self._widths)]

    # -- the native side --------------------------------------------------------

    def enter(self):
        """Before a native call: the stream that torch launches on now (a recording has its own)."""
        from ..ops import kernels

        self.c.stream = kernels.raw_stream()
        self.c.force_splits = kernels.force_splits
        return native.running(self)

    @property
    def read_ahead(self):
        return self._read_ahead

    @read_ahead.setter
    def read_ahead(self, w):
        """Weights (a ``PackedWeight``) that a kernel with idle CUs may read ahead, or ``None``."""
        self._read_ahead = w
        self.c.read_ahead = ctypes.pointer(w.c) if w is not None and hasattr(w, "c") else None

    _read_ahead = None

    def keep(self, *tensors):
        self._kept.extend(tensors)

    def tensor(self, m):
        """A torch tensor over the matrix ``m`` (an ``EngMat``) that the native side handed out."""
        dtype = native.TORCH_DT[m.dtype]
        es = 2 if dtype == torch.bfloat16 else 4
        n_bytes = ((m.rows - 1) * m.ld + m.cols) * es if m.rows > 0 else 0
        raw = self._scratch.view(m.p, n_bytes)
        if raw is None:
            logits = self.engine._logits
            if logits is not None:
                base = logits.data_ptr()
                if base <= m.p and m.p + n_bytes <= base + logits.numel() * 4:
                    raw = logits.view(-1).view(torch.uint8)[m.p - base : m.p - base + n_bytes]
        if raw is None:
            raw = torch.as_tensor(_DeviceArray(m.p, n_bytes), device=self.device)
        return torch.as_strided(raw.view(dtype), (m.rows, m.cols), (m.ld, 1))

    def int_array(self, p, n):
        """The int32 device array of ``n`` entries at address ``p`` (one of the step's own)."""
        if self._meta is not None:
            base = self._meta.data_ptr()
            if base <= p and p + 4 * n <= base + 4 * self._meta.numel():
                i = (p - base) // 4
                return self._meta[i : i + n]
        return torch.as_tensor(_DeviceArray(p, 4 * n), device=self.device).view(torch.int32)

    # -- what parts written in Python use -----------------------------------------

    def scratch(self, shape, dtype):
        return self._scratch.take(shape, dtype)

    def scratch_mark(self):
        return self._scratch.offset

    def scratch_release(self, mark):
        self._scratch.offset = mark

    def logits_out(self, n_rows, vocab):
        return self.engine.logits_buffer(n_rows, vocab)

    def cache_view(self, slot):
        v = self._views.get(slot)
        if v is None:
            cm = self.engine.cache
            if slot in cm.slot_group:
                from ..ops.kernels import PagedKV

                g, _ = cm.slot_group[slot]
                keys, values = cm.kv(slot)
                v = CacheView(slot, kv=PagedKV(keys, values) if keys.shape == values.shape else None,
                              block_table=self.block_tables[g], keys=keys, values=values)
            elif slot in cm.state_needs:
                v = CacheView(slot, state=cm.state(slot))
            else:
                v = CacheView(slot)
            self._views[slot] = v
        return v
