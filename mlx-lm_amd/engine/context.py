"""What a step's parts see: the flat batch on the device, cache views, scratch memory."""

import torch

_TORCH_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16, "int32": torch.int32}

ROW_KERNEL_MAX_Q = 4  # requests with at most this many tokens in a step take the row kernel
TILE_Q = 16  # queries per tile of the general tile kernel
BIG_TILE_Q = 128  # queries per tile of the matrix-core prefill kernel


class Scratch:
    """A bump allocator over one device buffer, reset at every step.

    The same sequence of requests gives the same addresses, so a step's
    launches can be recorded and replayed.  The buffer grows (outside of a
    recording) when a step needs more than any step before.
    """

    ALIGN = 256

    def __init__(self, device, initial_bytes=1 << 20):
        self.device = device
        self.buffer = torch.empty(initial_bytes, dtype=torch.uint8, device=device)
        self.offset = 0
        self.peak = 0
        self.frozen = False
        self._old = []  # outgrown buffers, kept alive until the next reset

    def reset(self):
        self.offset = 0
        self._old.clear()

    def take(self, shape, dtype):
        dtype = _TORCH_DTYPES.get(dtype, dtype)
        n = 1
        for s in shape:
            n *= int(s)
        nbytes = n * torch.empty((), dtype=dtype).element_size()
        start = (self.offset + self.ALIGN - 1) // self.ALIGN * self.ALIGN
        end = start + nbytes
        if end > self.buffer.numel():
            if self.frozen:
                raise RuntimeError("scratch memory would have to grow while a step is being recorded")
            # earlier views of this step stay valid: the old buffer is kept until reset
            self._old.append(self.buffer)
            self.buffer = torch.empty(max(end, 2 * self.buffer.numel()), dtype=torch.uint8,
                                      device=self.device)
        self.offset = end
        self.peak = max(self.peak, end)
        return self.buffer[start:end].view(dtype).view(*shape)


class CacheView:
    """One cache slot as a mixer sees it in a step."""

    __slots__ = ("kv", "block_table", "state", "slot")

    def __init__(self, slot, kv=None, block_table=None, state=None):
        self.slot, self.kv, self.block_table, self.state = slot, kv, block_table, state


class AttentionPlan:
    """Which of the step's rows go to which attention kernel.

    Requests that bring at most ``ROW_KERNEL_MAX_Q`` tokens are handled row by
    row (keys split over blocks); longer portions in tiles of ``TILE_Q``
    consecutive queries (``big_tiles``: the same portions in tiles of
    ``BIG_TILE_Q``, longest context first, for the matrix-core kernel).
    ``all_tiles`` covers every row with tiles, for mixers whose head size the
    row kernel does not take.
    """

    def __init__(self):
        self.tiles = self.rows = self.all_tiles = self.big_tiles = None
        self.n_tiles = self.n_rows = self.n_all_tiles = self.n_big_tiles = 0
        self.max_row_context = 0
        self.n_compute_units = 256

    def row_splits(self, n_heads, window=0):
        """How many ways to split a row's keys so that the launch fills the GPU."""
        ctx = self.max_row_context if window <= 0 else min(self.max_row_context, window + 63)
        most = max(1, (ctx + 255) // 256)  # a block's four waves want a tile each
        want = (2 * self.n_compute_units + self.n_rows * n_heads - 1) // max(1, self.n_rows * n_heads)
        return max(1, min(most, want, 64))

    def row_work(self, n_heads, window=0, max_waves=16):
        """``(n_splits, n_waves)`` for a decode kernel whose blocks take 2 to ``max_waves`` waves.

        Few rows: many waves a block (a tile of 64 keys each) keep the GPU busy
        without the second kernel that joining splits needs.  Many rows: few
        waves a block, each with several tiles, so that a block's fixed cost
        (its way to the first key, joining its waves) is spread over more keys.
        Splits only where sixteen waves would take three tiles or more each and
        the splits' blocks still find a compute unit each at once: measured, a
        split that has to wait for a compute unit costs more than the longer
        loop that it saves.
        """
        ctx = self.max_row_context if window <= 0 else min(self.max_row_context, window + 63)
        tiles = max(1, (ctx + 63) // 64)
        blocks = max(1, self.n_rows * n_heads)
        want = (8 * self.n_compute_units + blocks - 1) // blocks  # eight waves a CU in all
        n_waves = 2
        while n_waves < max_waves and n_waves < want and n_waves < tiles:
            n_waves *= 2
        rounds = (tiles + n_waves - 1) // n_waves
        n_splits = 1
        if rounds >= 3:
            n_splits = max(1, min(rounds, self.n_compute_units // blocks, 64))
        return n_splits, n_waves


class StepContext:
    """One step's batch, as the parts see it.

    Tokens of all requests lie in one flat list.  ``token_ids``, ``positions``
    and ``token_req`` (row of the request in the block tables) are int32
    device arrays over the tokens; ``slot_ids`` gives each request's state
    slot; ``wanted_rows`` the flat rows whose logits are asked for.  The host
    lists ``q_starts``/``q_lens``/``context_lens`` (tokens before this step)
    say where each request's run lies, ``state_slots`` is ``slot_ids`` on the host.
    """

    def __init__(self, engine):
        self.engine = engine
        self.dtype = engine.dtype
        self.device = engine.device
        self._scratch = engine.scratch
        self.n_tokens = self.n_requests = self.n_wanted = 0
        self.token_ids = self.positions = self.token_req = None
        self.slot_ids = self.wanted_rows = None
        self.block_tables = []
        self.q_starts, self.q_lens, self.context_lens, self.state_slots = [], [], [], []
        self.attention_plan = AttentionPlan()
        self._views = {}
        # a projection's sum into the residual stream that the next norm will add
        from ..ops.kernels import PendingSum

        self.pending = PendingSum()
        self.wants_every_row = False  # wanted_rows is 0 .. n_tokens - 1
        self.read_ahead = None  # weights (a PackedWeight) that a kernel with idle CUs may read ahead

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
                v = CacheView(slot, kv=PagedKV(*cm.kv(slot)), block_table=self.block_tables[g])
            elif slot in cm.state_needs:
                v = CacheView(slot, state=cm.state(slot))
            else:
                v = CacheView(slot)
            self._views[slot] = v
        return v
