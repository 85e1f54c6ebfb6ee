"""Pages of keys and values for every live request, and slots of fixed-size state.

The reference keeps one growing array per layer and request (``KVCache``,
mlx_lm/models/cache.py:325-407) or per layer and batch (``BatchKVCache``,
921-1139, batched by padding), sliding windows in ``RotatingKVCache``
(410-591) and fixed-size state in ``ArraysCache`` (594-733).  Here memory is
cut into pages of ``page_size`` tokens instead:

* Cache slots (one per layer run that writes a cache) whose mixers want the
  same thing -- same key heads, widths of a key and of a value, and window --
  form a *group*.  A
  group has one pool of pages; page ``p`` of the group is one page in every
  slot of the group, so a request has one block table per group.
* A request's block table lists, for block ``b`` (positions ``b*page_size ..``),
  the page that holds it, or -1 once a window has passed it.
* Pages are taken before a step runs (``reserve``) and counted as filled after
  it (``commit``); they are given back when the request ends (``release``), is
  cut short (``truncate``) or, in a windowed group, when every later query is
  out of their reach.
* Every request also gets a state slot: a row in each fixed-size state tensor
  (zeroed when the request starts), whether or not any mixer asks for one.
* What a request computed can be kept beyond its end (``detach``) for a later
  request to go on from (``attach``): its pages simply stay held.
"""

from dataclasses import dataclass, field
from typing import Dict, List

from ..config.plan import CacheNeed, StateNeed
from .pages import PagePool


class OutOfPages(RuntimeError):
    """Not enough free pages for what was asked."""


class OutOfSlots(RuntimeError):
    """Every state slot is taken."""


@dataclass
class RequestCache:
    request_id: object
    state_slot: int
    length: int = 0  # tokens whose keys and values are in the pages
    reserved: int = 0  # tokens that have pages (>= length)
    blocks: List[List[int]] = field(default_factory=list)  # per group: page of each block or -1
    serial: int = 0  # unique over the manager's life, unlike the id
    version: int = 0  # counts the edits of ``blocks``: who keeps a copy of a table compares it


@dataclass
class KeptPages:
    """What a request had computed, taken out of the list of live requests but not given back:
    its pages stay held (no other request gets them), its state rows are copied.  ``attach``
    makes a live request of it again, ``drop`` gives everything back.  (The reference keeps a
    request's arrays as its prompt cache, mlx_lm/models/cache.py:15-43; with pages nothing is copied.)"""

    length: int
    reserved: int
    blocks: List[List[int]]
    state: Dict[int, object] = field(default_factory=dict)  # cache slot -> the request's row of that state tensor
    live: bool = True  # False once attached again or dropped


class _Group:
    def __init__(self, need: CacheNeed, n_pages):
        self.need = need
        self.slots: List[int] = []
        self.pool = PagePool(n_pages)
        # keys [n_slots, n_pages, n_kv_heads, page_size, head_dim] and values [.., value_dim]: where both
        # have one width they are the two halves of every page of one tensor, keys first
        self.keys = self.values = None


class CacheManager:
    """Pages, block tables and state slots for the requests that are live.

    ``needs`` has one entry per cache slot: a ``CacheNeed``, a ``StateNeed`` or
    ``None``.  ``n_pages`` is the number of pages of every group.  With
    ``device`` set, storage is allocated there in ``dtype``; without, the
    manager only does the bookkeeping (for tests and dry runs).
    """

    def __init__(self, needs, page_size, n_pages, max_requests, dtype=None, device=None):
        if page_size <= 0 or page_size % 16:
            raise ValueError(f"page_size must be a positive multiple of 16, got {page_size}")
        if max_requests <= 0:
            raise ValueError("max_requests must be positive")
        self.page_size, self.n_pages, self.max_requests = page_size, n_pages, max_requests
        self.dtype, self.device = dtype, device
        self.groups: List[_Group] = []
        self.slot_group: Dict[int, tuple] = {}  # cache slot -> (group index, index in the group)
        self.state_needs: Dict[int, StateNeed] = {}
        self.state_storage: Dict[int, object] = {}
        by_need = {}
        for slot, need in enumerate(needs):
            if isinstance(need, CacheNeed):
                if need not in by_need:
                    by_need[need] = len(self.groups)
                    self.groups.append(_Group(need, n_pages))
                g = by_need[need]
                self.slot_group[slot] = (g, len(self.groups[g].slots))
                self.groups[g].slots.append(slot)
            elif isinstance(need, StateNeed):
                self.state_needs[slot] = need
            elif need is not None:
                raise TypeError(f"cache slot {slot}: unknown need {need!r}")
        self._free_state_slots = list(range(max_requests - 1, -1, -1))
        self.requests: Dict[object, RequestCache] = {}
        self.kept: List[KeptPages] = []  # detached and neither attached again nor dropped
        if device is not None:
            self._allocate()

    def _allocate(self):
        import torch

        for g in self.groups:
            n = g.need
            shape = (len(g.slots), self.n_pages, n.n_kv_heads, self.page_size)
            if n.value_dim == n.head_dim:
                # a page's keys and values side by side: one stride for both, which the attention
                # kernels here ask for
                both = torch.zeros((*shape[:2], 2, *shape[2:], n.head_dim), dtype=self.dtype, device=self.device)
                g.keys, g.values = both[:, :, 0], both[:, :, 1]
            else:
                g.keys = torch.zeros((*shape, n.head_dim), dtype=self.dtype, device=self.device)
                g.values = torch.zeros((*shape, n.value_dim), dtype=self.dtype, device=self.device)
        for slot, need in self.state_needs.items():
            self.state_storage[slot] = torch.zeros(
                (self.max_requests, *need.shape), dtype=getattr(torch, need.dtype), device=self.device
            )

    # -- sizes ---------------------------------------------------------------

    def blocks_for(self, n_tokens):
        return (n_tokens + self.page_size - 1) // self.page_size

    def bytes_per_token(self):
        """Bytes of keys and values that one token takes over all slots."""
        import torch

        size = torch.empty((), dtype=self.dtype).element_size() if self.dtype is not None else 0
        return sum(g.need.n_kv_heads * (g.need.head_dim + g.need.value_dim) * len(g.slots) * size
                   for g in self.groups)

    def free_pages(self):
        """Free pages of the group that has fewest."""
        return min((g.pool.n_free for g in self.groups), default=self.n_pages)

    def pages_needed(self, request_id, n_new):
        """Pages that ``reserve(request_id, n_new)`` would take (the most over the groups)."""
        rc = self.requests[request_id]
        return max(0, self.blocks_for(rc.length + n_new) - self.blocks_for(rc.reserved))

    # -- life of a request -----------------------------------------------------

    def add(self, request_id):
        if request_id in self.requests:
            raise ValueError(f"request {request_id!r} is already live")
        if not self._free_state_slots:
            raise OutOfSlots(f"all {self.max_requests} request slots are taken")
        slot = self._free_state_slots.pop()
        self._serial = getattr(self, "_serial", 0) + 1
        rc = RequestCache(request_id, slot, blocks=[[] for _ in self.groups], serial=self._serial)
        self.requests[request_id] = rc
        for storage in self.state_storage.values():
            storage[slot].zero_()
        return rc

    def reserve(self, request_id, n_new):
        """Make sure positions ``length .. length+n_new-1`` have pages in every group.

        All or nothing: if any group is short, nothing is taken and
        ``OutOfPages`` is raised.
        """
        rc = self.requests[request_id]
        if n_new < 0:
            raise ValueError("cannot reserve a negative number of tokens")
        want_blocks = self.blocks_for(rc.length + n_new)
        taken = []
        for gi, g in enumerate(self.groups):
            extra = want_blocks - len(rc.blocks[gi])
            pages = g.pool.take(extra) if extra > 0 else []
            if pages is None:
                for gj, got in taken:
                    self.groups[gj].pool.give_back(got)
                raise OutOfPages(
                    f"request {request_id!r} needs {extra} more pages, {g.pool.n_free} are free"
                )
            taken.append((gi, pages))
        for gi, pages in taken:
            if pages:
                rc.blocks[gi].extend(pages)
                rc.version += 1
        rc.reserved = max(rc.reserved, rc.length + n_new)
        return rc

    def mark(self, request_id):
        """What ``rollback`` needs to undo the reservations that follow."""
        rc = self.requests[request_id]
        return (rc.reserved, [len(b) for b in rc.blocks])

    def rollback(self, request_id, mark):
        """Give back the pages taken since ``mark`` (a step that could not get all its pages):
        what the request held before, filled or only reserved, stays its own."""
        rc = self.requests[request_id]
        reserved, n_blocks = mark
        for gi, g in enumerate(self.groups):
            extra = [p for p in rc.blocks[gi][n_blocks[gi]:] if p >= 0]
            if len(rc.blocks[gi]) > n_blocks[gi]:
                g.pool.give_back(extra)
                del rc.blocks[gi][n_blocks[gi]:]
                rc.version += 1
        rc.reserved = reserved
        return rc

    def commit(self, request_id, n_new):
        """Count ``n_new`` more tokens as stored; give back pages a window has passed."""
        rc = self.requests[request_id]
        if rc.length + n_new > rc.reserved:
            raise ValueError(f"request {request_id!r}: committing tokens that were never reserved")
        rc.length += n_new
        for gi, g in enumerate(self.groups):
            w = g.need.window
            if w <= 0:
                continue
            # the next query sits at position >= length and sees keys > position - w
            first_needed = max(0, rc.length - w + 1)
            for b in range(first_needed // self.page_size):
                if rc.blocks[gi][b] >= 0:
                    g.pool.give_back([rc.blocks[gi][b]])
                    rc.blocks[gi][b] = -1
                    rc.version += 1
        return rc

    def truncate(self, request_id, new_length):
        """Forget the tokens from ``new_length`` on (``trim`` of mlx_lm/models/cache.py:378-381).

        Whole pages beyond the new end go back.  A windowed group that has
        already given back pages the shorter sequence would need again cannot
        be truncated.
        """
        rc = self.requests[request_id]
        if not (0 <= new_length <= rc.length):
            raise ValueError(f"cannot truncate request {request_id!r} from {rc.length} to {new_length}")
        keep = self.blocks_for(new_length)
        for gi, g in enumerate(self.groups):
            w = g.need.window
            if w > 0:
                first_needed = max(0, new_length - w + 1) // self.page_size
                if any(p < 0 for p in rc.blocks[gi][first_needed:keep]):
                    raise ValueError(
                        f"request {request_id!r}: a window has already dropped pages that "
                        f"length {new_length} needs"
                    )
        for gi, g in enumerate(self.groups):
            tail = [p for p in rc.blocks[gi][keep:] if p >= 0]
            g.pool.give_back(tail)
            del rc.blocks[gi][keep:]
        rc.version += 1
        rc.length = new_length
        rc.reserved = min(rc.reserved, keep * self.page_size)
        rc.reserved = max(rc.reserved, rc.length)
        return rc

    def release(self, request_id):
        """The request is over: all its pages and its state slot go back."""
        rc = self.requests.pop(request_id)
        for gi, g in enumerate(self.groups):
            g.pool.give_back([p for p in rc.blocks[gi] if p >= 0])
        self._free_state_slots.append(rc.state_slot)

    # -- keeping what a request computed ----------------------------------------

    def detach(self, request_id):
        """Take a request out and keep what it holds: its pages stay held, its state rows are
        copied, its request slot goes back.  Returns the ``KeptPages``."""
        rc = self.requests.pop(request_id)
        state = {slot: storage[rc.state_slot].clone() for slot, storage in self.state_storage.items()}
        self._free_state_slots.append(rc.state_slot)
        kept = KeptPages(rc.length, rc.reserved, rc.blocks, state)
        self.kept.append(kept)
        return kept

    def attach(self, request_id, kept):
        """A live request that goes on from what ``kept`` holds (which is used up by this)."""
        if not kept.live or not any(k is kept for k in self.kept):
            raise ValueError("these kept pages are not this cache manager's, or were used already")
        rc = self.add(request_id)
        rc.length, rc.reserved, rc.blocks = kept.length, kept.reserved, kept.blocks
        rc.version += 1
        for slot, row in kept.state.items():
            self.state_storage[slot][rc.state_slot].copy_(row)
        self._forget(kept)
        return rc

    def fork(self, kept):
        """A second ``KeptPages`` with the same tokens in pages of its own (their contents are
        copied on the device), so that two requests can go on from one point.  All or nothing:
        ``OutOfPages`` if a group is short."""
        if not kept.live:
            raise ValueError("these kept pages were used already")
        n_blocks = self.blocks_for(kept.length)
        taken = []
        for gi, g in enumerate(self.groups):
            old = kept.blocks[gi][:n_blocks]
            new = g.pool.take(sum(p >= 0 for p in old))
            if new is None:
                for gj, pages in taken:
                    self.groups[gj].pool.give_back(pages)
                raise OutOfPages(f"a copy of {kept.length} kept tokens needs {sum(p >= 0 for p in old)} pages "
                                 f"of group {gi}; {g.pool.n_free} are free")
            taken.append((gi, new))
        blocks = []
        for (gi, new), g in zip(taken, self.groups):
            old = kept.blocks[gi][:n_blocks]
            fresh = iter(new)
            blocks.append([next(fresh) if p >= 0 else -1 for p in old])
            src = [p for p in old if p >= 0]
            if g.keys is not None and src:
                import torch

                i_src = torch.tensor(src, device=g.keys.device)
                i_dst = torch.tensor(new, device=g.keys.device)
                g.keys.index_copy_(1, i_dst, g.keys.index_select(1, i_src))
                g.values.index_copy_(1, i_dst, g.values.index_select(1, i_src))
        state = {slot: row.clone() for slot, row in kept.state.items()}
        copy = KeptPages(kept.length, n_blocks * self.page_size, blocks, state)
        self.kept.append(copy)
        return copy

    def read_kept(self, kept):
        """What a ``KeptPages`` holds, out of its pages: ``({slot: (keys [tokens, n_kv_heads,
        head_dim], values [tokens, n_kv_heads, value_dim])}, {slot: state row})`` as tensors of
        their own (for a file, or for another engine's pool)."""
        import torch

        if not kept.live:
            raise ValueError("these kept pages were used already")
        n_blocks = self.blocks_for(kept.length)
        out = {}
        for gi, g in enumerate(self.groups):
            pages = kept.blocks[gi][:n_blocks]
            if any(p < 0 for p in pages):
                raise ValueError("a window has given pages of these tokens back: what is left cannot "
                                 "stand for the tokens and is not written out")
            index = torch.tensor(pages, dtype=torch.long, device=g.keys.device)
            for i, slot in enumerate(g.slots):
                both = []
                for pool in (g.keys[i], g.values[i]):  # [pages, heads, page, width]
                    t = pool.index_select(0, index).permute(0, 2, 1, 3)
                    both.append(t.reshape(-1, t.shape[2], t.shape[3])[: kept.length].contiguous())
                out[slot] = tuple(both)
        return out, {slot: row.clone() for slot, row in kept.state.items()}

    def write_kept(self, length, per_slot, state):
        """The opposite of ``read_kept``: pages of this pool filled with the given keys and values.
        Returns the ``KeptPages`` (``OutOfPages`` if the pool is short, with nothing taken)."""
        import torch

        if set(per_slot) != set(self.slot_group) or set(state) != set(self.state_needs):
            raise ValueError(f"the cache was written by a model with other layers: it has the cache slots "
                             f"{sorted(per_slot)} and state slots {sorted(state)}, this model "
                             f"{sorted(self.slot_group)} and {sorted(self.state_needs)}")
        for slot, (k, v) in per_slot.items():
            g = self.groups[self.slot_group[slot][0]]
            want_k = (length, g.need.n_kv_heads, g.need.head_dim)
            want_v = (length, g.need.n_kv_heads, g.need.value_dim)
            if tuple(k.shape) != want_k or tuple(v.shape) != want_v:
                raise ValueError(f"cache slot {slot}: keys {tuple(k.shape)} and values {tuple(v.shape)} in the "
                                 f"cache, {want_k} and {want_v} in this model")
        for slot, row in state.items():
            if tuple(row.shape) != tuple(self.state_storage[slot].shape[1:]):
                raise ValueError(f"state slot {slot}: shape {tuple(row.shape)} in the cache, "
                                 f"{tuple(self.state_storage[slot].shape[1:])} in this model")
        n_blocks = self.blocks_for(length)
        taken = []
        for gi, g in enumerate(self.groups):
            pages = g.pool.take(n_blocks)
            if pages is None:
                for gj, got in taken:
                    self.groups[gj].pool.give_back(got)
                raise OutOfPages(f"a cache of {length} tokens needs {n_blocks} pages of group {gi}; "
                                 f"{g.pool.n_free} are free")
            taken.append((gi, pages))
        blocks = []
        for (gi, pages), g in zip(taken, self.groups):
            blocks.append(pages)
            index = torch.tensor(pages, dtype=torch.long, device=g.keys.device)
            for i, slot in enumerate(g.slots):
                for pool, t in zip((g.keys[i], g.values[i]), per_slot[slot]):
                    full = torch.zeros((n_blocks * self.page_size, *t.shape[1:]), dtype=pool.dtype, device=pool.device)
                    full[:length] = t.to(device=pool.device, dtype=pool.dtype)
                    full = full.view(n_blocks, self.page_size, *t.shape[1:]).permute(0, 2, 1, 3)
                    pool.index_copy_(0, index, full)
        rows = {slot: row.to(device=self.state_storage[slot].device, dtype=self.state_storage[slot].dtype).clone()
                for slot, row in state.items()}
        kept = KeptPages(length, n_blocks * self.page_size, blocks, rows)
        self.kept.append(kept)
        return kept

    def set_state(self, request_id, state=None):
        """A live request's rows of the state tensors: as ``state`` (cache slot -> row) has them, or zero."""
        rc = self.requests[request_id]
        for slot, storage in self.state_storage.items():
            if state is None:
                storage[rc.state_slot].zero_()
            else:
                storage[rc.state_slot].copy_(state[slot])

    def drop(self, kept):
        """Give back the pages of a ``KeptPages`` that nobody goes on from."""
        if not kept.live:
            return
        for gi, g in enumerate(self.groups):
            g.pool.give_back([p for p in kept.blocks[gi] if p >= 0])
        self._forget(kept)

    def _forget(self, kept):
        kept.live = False
        self.kept = [k for k in self.kept if k is not kept]

    def truncate_kept(self, kept, new_length):
        """``truncate`` for pages that are kept: forget the tokens from ``new_length`` on.  (State rows
        cannot be taken back; whether a model's state allows a cut is the caller's to know.)"""
        if not kept.live:
            raise ValueError("these kept pages were used already")
        # (through a request of a moment: the rules are truncate's)
        name = ("kept", id(kept))
        rc = RequestCache(name, -1, kept.length, kept.reserved, kept.blocks)
        self.requests[name] = rc
        try:
            self.truncate(name, new_length)
        finally:
            del self.requests[name]
        kept.length, kept.reserved, kept.blocks = rc.length, rc.reserved, rc.blocks
        return kept

    def release_all(self):
        for rid in list(self.requests):
            self.release(rid)

    # -- views for a step ------------------------------------------------------

    def block_table(self, request_id, group):
        return self.requests[request_id].blocks[group]

    def kv(self, slot):
        """``(keys, values)`` of cache slot ``slot``: ``[n_pages, n_kv_heads, page, head_dim]`` and
        ``[.., value_dim]``."""
        g, i = self.slot_group[slot]
        return self.groups[g].keys[i], self.groups[g].values[i]

    def state(self, slot):
        """State tensor of cache slot ``slot``: ``[max_requests, *shape]``."""
        return self.state_storage[slot]

    def poison_free_pages(self, value=float("nan")):
        """Overwrite every page that no request holds (tests: stale pages must not matter)."""
        import torch

        for g in self.groups:
            free = torch.tensor(sorted(g.pool._free), dtype=torch.long, device=g.keys.device)
            if free.numel():
                g.keys[:, free] = value
                g.values[:, free] = value

    def check(self):
        """No page lost, held twice or free while in a block table."""
        for gi, g in enumerate(self.groups):
            g.pool.check()
            seen = {}
            holders = [(rc.request_id, rc.blocks) for rc in self.requests.values()]
            holders += [(("kept", i), k.blocks) for i, k in enumerate(self.kept)]
            for holder, blocks in holders:
                for p in blocks[gi]:
                    if p < 0:
                        continue
                    if p in seen:
                        raise AssertionError(f"group {gi}: page {p} held by {seen[p]!r} and {holder!r}")
                    if not g.pool._held[p]:
                        raise AssertionError(f"group {gi}: page {p} in a block table but free")
                    seen[p] = holder
            if len(seen) != g.pool.n_held:
                raise AssertionError(
                    f"group {gi}: {g.pool.n_held} pages held but {len(seen)} in block tables"
                )
        slots = [rc.state_slot for rc in self.requests.values()]
        if len(set(slots)) != len(slots) or set(slots) & set(self._free_state_slots):
            raise AssertionError("a state slot is held twice or both held and free")
        if len(slots) + len(self._free_state_slots) != self.max_requests:
            raise AssertionError("a state slot is lost")
