"""What a request has computed, kept for a later request to go on from.

The reference keeps a list of per-layer caches (``make_prompt_cache``,
mlx_lm/models/cache.py:15-43) that ``generate_step(..., prompt_cache=...)``
fills and updates in place (mlx_lm/generate.py:306,329-331,362-385), that
``trim_prompt_cache`` shortens (mlx_lm/models/cache.py:88-111) and that
``BatchGenerator`` takes and hands back per request
(mlx_lm/generate.py:1689-1731,1777-1802).  Here a kept cache is one object for
the whole model: the pages that the request held in the engine's pool, which
simply stay held, and the request's row of every state tensor.  Nothing is
copied when a request goes on from it.  ``save_prompt_cache`` writes the keys,
values and state out of the pages into a safetensors file and
``load_prompt_cache`` reads them back (mlx_lm/models/cache.py:43-85); a cache
that was read from a file holds tensors of its own until the first request
that uses it gives it pages in that request's engine.
"""

import json


class PromptCache:
    """Keys, values and state of the tokens that went through it, in the pool of one engine.

    A request is given it as ``prompt_cache`` (``generate_step``, ``stream_generate``) or in
    ``caches`` (``BatchGenerator.insert``); it then reads only the tokens it brings, on top
    of what the cache holds, and when it ends the cache holds those tokens and all the
    generated ones as well (the very last one as ``pending``: it has not gone through the model,
    the next request reads it first).  While a request uses it, nobody else can.  ``offset`` is
    the number of tokens held.  The pages count against the engine's pool until ``free()`` (or
    until the object goes away).
    """

    def __init__(self, model=None):
        self.model = model
        self._engine = None
        self._kept = None
        # (length, {slot: (keys, values)}, {slot: state row}) of a cache that was read from a file
        # and has no pages yet
        self._loaded = None
        self._at_checkout = (0, None)
        self.in_use = False    # a live request holds the pages
        self.claimed = False   # a request that waits or runs will go on from this cache
        # Tokens that belong to the cache but have not gone through the model: the token that
        # ended the request before (it ends a request before it is fed).  The next request reads
        # them ahead of its prompt.
        self.pending = []

    @property
    def offset(self):
        """Tokens held, the pending ones included."""
        if self._kept is not None:
            in_pages = self._kept.length
        else:
            in_pages = self._loaded[0] if self._loaded is not None else 0
        return in_pages + len(self.pending)

    @property
    def needs_pages(self):
        """Read from a file and not yet in any engine's pool: the first request brings it there."""
        return self._loaded is not None

    @property
    def engine(self):
        """The engine in whose pool the tokens lie (``None`` while the cache is empty and was never used)."""
        return self._engine if (self._kept is not None or self.in_use) else None

    def __len__(self):
        return self.offset

    # -- what the scheduler calls ------------------------------------------------

    def checkout(self, engine, engine_id):
        """A live request ``engine_id`` of ``engine`` that holds what this cache holds."""
        if self.in_use:
            raise ValueError("this prompt cache is in use by a live request")
        if self._kept is not None and self._engine is not engine:
            raise ValueError("this prompt cache holds pages of another engine (another cache geometry or model)")
        if self._loaded is not None:  # read from a file: into pages of this engine's pool now
            self._kept = engine.write_kept(*self._loaded)
            self._loaded, self._engine = None, engine
        at_checkout = (self.offset - len(self.pending), self._kept.state if self._kept is not None else None)
        if self._kept is None:
            engine.add_request(engine_id)  # (may find no request slot free: nothing has changed then)
        else:
            engine.attach_request(engine_id, self._kept)
            self._kept = None
        self._engine, self.in_use, self._at_checkout = engine, True, at_checkout
        self.pending = []  # (the request has them: it reads them ahead of its prompt)

    def rewind(self, engine, engine_id, length=None):
        """Cut the live request back to ``length`` tokens, or to what the cache held when the request
        took it.  Per-request state cannot be cut: a model that has some goes all the way back,
        its state rows as they were then."""
        offset, state = self._at_checkout
        if length is None or (engine.cache.state_needs and length != engine.context_len(engine_id)):
            length = offset
            if engine.cache.state_needs:
                engine.cache.set_state(engine_id, state)
        engine.cache.truncate(engine_id, length)

    def checkin(self, engine, engine_id):
        """The request ends: what it holds is this cache's from now on."""
        self._engine = engine
        # pages taken ahead of the tokens go back (the cache manager's own cut: no token is dropped)
        engine.cache.truncate(engine_id, engine.context_len(engine_id))
        self._kept = engine.detach_request(engine_id)
        self.in_use = False

    # -- what callers use ----------------------------------------------------------

    def is_trimmable(self):
        if self.in_use or self.claimed:
            return False
        if self._loaded is not None:
            return not self._loaded[2]
        return self._engine is None or not self._engine.cache.state_needs

    def trim(self, n_tokens):
        """Forget the last ``n_tokens`` tokens (at most all); returns how many went."""
        if self.in_use or self.claimed:
            raise ValueError("this prompt cache is in use by a request")
        n = max(0, min(int(n_tokens), self.offset))
        first = min(n, len(self.pending))  # the tokens that are not in pages yet go first
        self.pending = self.pending[: len(self.pending) - first]
        rest = n - first
        if rest and self._loaded is not None:
            length, per_slot, state = self._loaded
            self._loaded = (length - rest, {s: (k[: length - rest], v[: length - rest]) for s, (k, v) in per_slot.items()}, state)
        elif rest:
            self._engine.cache.truncate_kept(self._kept, self._kept.length - rest)
        return n

    def copy(self):
        """A second cache with the same tokens, in pages of its own (``OutOfPages`` if the pool is short)."""
        if self.in_use:
            raise ValueError("this prompt cache is in use by a live request")
        other = PromptCache(self.model)
        other.pending = list(self.pending)
        other._loaded = self._loaded  # (never written to: trim makes a new tuple)
        if self._kept is not None:
            other._engine = self._engine
            other._kept = self._engine.cache.fork(self._kept)
        return other

    def tensors(self):
        """``(length, {slot: (keys, values)}, {slot: state row})``: the tokens' keys ``[length,
        n_kv_heads, head_dim]`` and values of every cache slot and the state rows, as tensors of
        their own."""
        if self.in_use:
            raise ValueError("this prompt cache is in use by a live request")
        if self._loaded is not None:
            return self._loaded
        if self._kept is None:
            return 0, {}, {}
        per_slot, state = self._engine.read_kept(self._kept)
        return self._kept.length, per_slot, state

    def free(self):
        """Give the pages back to the engine's pool; the cache is empty afterwards."""
        self._loaded = None
        if not self.in_use:
            self.pending = []
        if self._kept is not None and not self.in_use:
            self._engine.drop_kept(self._kept)
            self._kept = None

    def __del__(self):
        try:
            self.free()
        except Exception:  # noqa: BLE001 (the interpreter may be shutting down)
            pass


def make_prompt_cache(model=None, max_kv_size=None):
    """An empty cache for ``model`` (``make_prompt_cache`` of mlx_lm/models/cache.py:15-43)."""
    if max_kv_size is not None:
        raise ValueError("'max_kv_size' is not supported by this engine")
    return PromptCache(model)


_FORMAT = "mlx_lm_amd prompt cache 1"


def save_prompt_cache(file_name, cache, metadata=None):
    """Write a cache's keys, values and state rows to a ``.safetensors`` file, with ``metadata``
    (a dict of strings) beside them (``save_prompt_cache`` of mlx_lm/models/cache.py:43-59)."""
    from safetensors.torch import save_file

    length, per_slot, state = cache.tensors()
    tensors = {}
    for slot, (k, v) in per_slot.items():
        tensors[f"slot.{slot}.keys"] = k.detach().cpu().contiguous()
        tensors[f"slot.{slot}.values"] = v.detach().cpu().contiguous()
    for slot, row in state.items():
        tensors[f"state.{slot}"] = row.detach().cpu().contiguous()
    if not tensors:  # (a file of no tensors: an empty cache is one tensor of nothing)
        import torch

        tensors["empty"] = torch.zeros(0)
    info = {"format": _FORMAT, "length": str(int(length)), "pending": json.dumps([int(t) for t in cache.pending]),
            "metadata": json.dumps({str(k): str(v) for k, v in (metadata or {}).items()})}
    save_file(tensors, file_name, metadata=info)


def load_prompt_cache(file_name, return_metadata=False):
    """Read a cache that ``save_prompt_cache`` wrote (``load_prompt_cache`` of
    mlx_lm/models/cache.py:62-85).  Its tensors get pages in the engine of the first request that
    uses it, which must be of a model with the same layers, heads and head sizes."""
    from safetensors import safe_open

    per_slot, state = {}, {}
    with safe_open(file_name, framework="pt", device="cpu") as fh:
        info = fh.metadata() or {}
        if info.get("format") != _FORMAT:
            raise ValueError(f"{file_name} is not a prompt cache of this engine (format {info.get('format')!r})")
        length = int(info["length"])
        for name in fh.keys():
            kind, _, rest = name.partition(".")
            if kind == "slot":
                slot, _, what = rest.partition(".")
                per_slot.setdefault(int(slot), {})[what] = fh.get_tensor(name)
            elif kind == "state":
                state[int(rest)] = fh.get_tensor(name)
    cache = PromptCache()
    if length or state:
        cache._loaded = (length, {slot: (kv["keys"], kv["values"]) for slot, kv in per_slot.items()}, state)
    cache.pending = [int(t) for t in json.loads(info.get("pending", "[]"))]
    metadata = json.loads(info.get("metadata", "{}"))
    return (cache, metadata) if return_metadata else cache


def can_trim_prompt_cache(cache):
    """mlx_lm/models/cache.py:88-92."""
    return cache.is_trimmable()


def trim_prompt_cache(cache, num_tokens):
    """Trim in place; returns the number of tokens trimmed (mlx_lm/models/cache.py:95-111)."""
    if not can_trim_prompt_cache(cache):
        return 0
    return cache.trim(num_tokens)
