"""The cache manager's bookkeeping (no GPU): no page lost, held twice or freed twice."""

import random

import pytest

from mlx_lm_amd.cache import CacheManager, OutOfPages, OutOfSlots, PagePool
from mlx_lm_amd.config import CacheNeed, StateNeed


def test_page_pool_is_lifo_and_strict():
    pool = PagePool(4)
    assert pool.take(2) == [0, 1] and pool.n_free == 2
    pool.give_back([0])
    assert pool.take(1) == [0]  # the page just given back comes out first
    assert pool.take(3) is None and pool.n_free == 2  # nothing taken when short
    with pytest.raises(ValueError, match="not held"):
        pool.give_back([3])
    pool.give_back([1])
    with pytest.raises(ValueError, match="not held"):
        pool.give_back([1])
    with pytest.raises(ValueError, match="not of this pool"):
        pool.give_back([9])
    pool.check()
    assert pool.high_water == 2


def _manager(n_pages=8, window=0, max_requests=4):
    needs = [CacheNeed(2, 16, 0), CacheNeed(2, 16, 0), CacheNeed(2, 16, window), None, StateNeed((3,))]
    return CacheManager(needs, 16, n_pages, max_requests)


def test_groups_follow_needs():
    cm = _manager(window=40)
    assert len(cm.groups) == 2 and cm.groups[0].slots == [0, 1] and cm.groups[1].slots == [2]
    assert cm.slot_group[2] == (1, 0) and 4 in cm.state_needs and 3 not in cm.slot_group
    assert len(_manager(window=0).groups) == 1


def test_reserve_commit_release():
    cm = _manager()
    a = cm.add("a")
    cm.reserve("a", 17)
    assert a.blocks[0] == [0, 1] and a.length == 0 and cm.free_pages() == 6
    cm.commit("a", 17)
    cm.reserve("a", 15)  # fits the second page
    assert cm.free_pages() == 6 and cm.pages_needed("a", 16) == 1
    cm.commit("a", 15)
    with pytest.raises(ValueError, match="never reserved"):
        cm.commit("a", 1)
    b = cm.add("b")
    with pytest.raises(OutOfPages):
        cm.reserve("b", 16 * 7)
    assert b.blocks[0] == [] and cm.free_pages() == 6  # all or nothing
    cm.release("a")
    assert cm.free_pages() == 8
    cm.reserve("b", 5)
    assert b.blocks[0] == [1]  # used again at once
    cm.check()
    with pytest.raises(ValueError, match="already live"):
        cm.add("b")


def test_state_slots():
    cm = _manager(max_requests=2)
    s0, s1 = cm.add("a").state_slot, cm.add("b").state_slot
    assert {s0, s1} == {0, 1}
    with pytest.raises(OutOfSlots):
        cm.add("c")
    cm.release("a")
    assert cm.add("c").state_slot == s0
    cm.check()


def test_window_gives_pages_back_as_it_passes():
    cm = _manager(n_pages=8, window=20)
    rc = cm.add("a")
    cm.reserve("a", 40)
    cm.commit("a", 40)
    # the next query is at 40 and sees keys 21..40: block 0 (0..15) is out of reach
    assert rc.blocks[1] == [-1, 1, 2] and rc.blocks[0] == [0, 1, 2]
    assert cm.groups[1].pool.n_free == 6
    for _ in range(30):
        cm.reserve("a", 1)
        cm.commit("a", 1)
    assert rc.length == 70 and [p >= 0 for p in rc.blocks[1]] == [False, False, False, True, True]
    cm.check()
    with pytest.raises(ValueError, match="window"):
        cm.truncate("a", 30)
    cm.truncate("a", 68)  # the query at 68 sees keys from 49 on: block 3 is still there
    assert len(rc.blocks[0]) == 5 and rc.length == 68
    with pytest.raises(ValueError, match="window"):
        cm.truncate("a", 66)  # would need key 47 again, whose page is gone
    cm.release("a")
    assert cm.free_pages() == 8


def test_truncate_gives_whole_pages_back():
    cm = _manager()
    rc = cm.add("a")
    cm.reserve("a", 50)
    cm.commit("a", 50)
    cm.truncate("a", 33)
    assert rc.length == 33 and len(rc.blocks[0]) == 3 and cm.free_pages() == 5
    cm.truncate("a", 32)
    assert len(rc.blocks[0]) == 2
    cm.reserve("a", 20)
    assert len(rc.blocks[0]) == 4
    cm.check()


@pytest.mark.parametrize("seed", range(6))
@pytest.mark.parametrize("window", [0, 24])
def test_random_orders_keep_every_page_accounted(seed, window):
    rng = random.Random(seed)
    cm = _manager(n_pages=12, window=window, max_requests=5)
    live, n, kept = {}, 0, []
    for _ in range(600):
        op = rng.random()
        if op < 0.08 and live:  # a request's pages are kept aside ...
            rid = rng.choice(list(live))
            kept.append((cm.detach(rid), live.pop(rid)))
            assert rid not in cm.requests
        elif op < 0.16 and kept:  # ... and go on under a new name, are cut back, or are given back
            k, length = kept.pop(rng.randrange(len(kept)))
            what = rng.random()
            if what < 0.5 and len(live) < 5:
                rid = f"r{n}"
                n += 1
                assert cm.attach(rid, k).length == length
                live[rid] = length
                with pytest.raises(ValueError):
                    cm.attach("again", k)
            elif what < 0.75 and window == 0:
                new = rng.randint(0, length)
                cm.truncate_kept(k, new)
                kept.append((k, new))
            elif what < 0.85:
                kept.append((k, length))
                try:
                    kept.append((cm.fork(k), length))
                except OutOfPages:
                    pass
            else:
                cm.drop(k)
                cm.drop(k)  # a second time is nothing
        elif op < 0.3 and len(live) < 5:
            rid = f"r{n}"
            n += 1
            cm.add(rid)
            live[rid] = 0
        elif op < 0.75 and live:
            rid = rng.choice(list(live))
            k = rng.choice([1, 1, 1, 2, 7, 16, 33])
            try:
                cm.reserve(rid, k)
            except OutOfPages:
                before = [g.pool.n_free for g in cm.groups]
                cm.check()
                assert before == [g.pool.n_free for g in cm.groups]
                continue
            if rng.random() < 0.9:
                cm.commit(rid, k)
                live[rid] += k
        elif op < 0.85 and live:
            rid = rng.choice(list(live))
            if window == 0:
                new = rng.randint(0, live[rid])
                cm.truncate(rid, new)
                live[rid] = new
        elif live:
            rid = rng.choice(list(live))
            cm.release(rid)
            del live[rid]
        cm.check()
        for rid, length in live.items():
            rc = cm.requests[rid]
            assert rc.length == length
            # every position a later query can see has a page
            lo = 0 if window == 0 else max(0, length - window + 1)
            for gi, g in enumerate(cm.groups):
                first = 0 if g.need.window == 0 else lo // 16
                assert all(p >= 0 for p in rc.blocks[gi][first : cm.blocks_for(length)])
    cm.release_all()
    assert all(g.pool.n_free == 12 - sum(sum(p >= 0 for p in k.blocks[gi]) for k, _ in kept)
               for gi, g in enumerate(cm.groups))
    for k, _ in kept:
        cm.drop(k)
    assert all(g.pool.n_free == 12 for g in cm.groups) and not cm.kept
    cm.check()


def test_every_edit_of_a_table_counts_its_version_up():
    """Whoever keeps a copy of a request's block table compares versions: a table that was cut
    and has grown back to its old number of pages is not the table it was."""
    cm = _manager()
    rc = cm.add("a")
    cm.reserve("a", 50)
    cm.commit("a", 50)
    v0, pages0 = rc.version, list(rc.blocks[0])
    cm.reserve("a", 1)  # no new page: the table is the same
    assert rc.version == v0
    cm.truncate("a", 30)
    v1 = rc.version
    assert v1 > v0
    other = cm.add("b")
    cm.reserve("b", 16)  # takes the page that "a" gave back last (the pool is a stack)
    cm.reserve("a", 34)
    assert len(rc.blocks[0]) == len(pages0) and rc.blocks[0] != pages0 and rc.version > v1
    assert set(other.blocks[0]) & set(pages0)
    cm.check()


def test_a_window_passing_a_page_counts_the_version_up():
    cm = _manager(window=24)
    rc = cm.add("a")
    cm.reserve("a", 40)
    v = rc.version
    cm.commit("a", 40)  # the first page is out of every later query's reach
    assert rc.blocks[1][0] == -1 and rc.blocks[0][0] >= 0 and rc.version > v


def test_rollback_gives_back_what_was_taken_since_the_mark_and_nothing_else():
    cm = _manager()
    rc = cm.add("a")
    cm.reserve("a", 60)  # a whole prompt's pages, taken at admission
    cm.commit("a", 10)
    mark = cm.mark("a")
    held = list(rc.blocks[0])
    cm.reserve("a", 70)  # one page more
    assert len(rc.blocks[0]) == len(held) + 1
    cm.rollback("a", mark)
    assert rc.blocks[0] == held and rc.reserved == 60 and rc.length == 10
    assert cm.free_pages() == 8 - len(held)
    cm.check()


def test_keys_and_values_may_differ_in_width():
    """A mixer may keep values of another width than its keys (``CacheNeed.v_head_dim``): such slots
    form a group of their own, keys and values are tensors of their own there, and both widths count
    in the bytes of a token.  With one width a page's keys and values lie side by side under one
    page stride, which the attention kernels ask for."""
    import torch

    same, narrow = CacheNeed(2, 32, 0), CacheNeed(2, 32, 0, v_head_dim=16)
    assert same != narrow and same.value_dim == 32 and narrow.value_dim == 16
    cm = CacheManager([same, narrow, narrow, same], 16, 5, 2, dtype=torch.bfloat16, device="cpu")
    assert len(cm.groups) == 2 and cm.slot_group[1][0] == cm.slot_group[2][0] != cm.slot_group[0][0]
    k, v = cm.kv(0)
    assert k.shape == v.shape == (5, 2, 16, 32) and k.stride(0) == v.stride(0) == 2 * 2 * 16 * 32
    assert v.data_ptr() - k.data_ptr() == 2 * 16 * 32 * 2  # the values follow the page's keys
    k, v = cm.kv(2)
    assert k.shape == (5, 2, 16, 32) and v.shape == (5, 2, 16, 16) and k.stride(0) != v.stride(0)
    assert cm.bytes_per_token() == 2 * (2 * 2 * (32 + 32) + 2 * 2 * (32 + 16))
    cm.add("r")
    cm.reserve("r", 20)
    cm.commit("r", 20)
    cm.poison_free_pages(7.0)
    held = set(cm.block_table("r", cm.slot_group[2][0]))
    k, v = cm.kv(2)
    for p in range(5):
        assert bool((k[p] == 7).all()) == (p not in held) and bool((v[p] == 7).all()) == (p not in held)
    cm.check()


def test_kept_pages_carry_contents_and_state():
    """``detach``/``attach`` move nothing but the state rows; ``fork`` copies the pages' contents into
    pages of its own (a window's missing pages stay missing) and fails whole when the pool is short."""
    import torch

    needs = [CacheNeed(2, 16, 0), CacheNeed(1, 16, 24, v_head_dim=32), StateNeed((3,))]
    cm = CacheManager(needs, 16, 9, 3, dtype=torch.float32, device="cpu")
    cm.add("a")
    cm.reserve("a", 70)
    cm.commit("a", 70)  # five blocks; the window of 24 has passed the first two
    rc = cm.requests["a"]
    assert rc.blocks[1][:2] == [-1, -1] and all(p >= 0 for p in rc.blocks[0])
    for gi, g in enumerate(cm.groups):
        for b, p in enumerate(rc.blocks[gi]):
            if p >= 0:
                g.keys[:, p] = 100 * gi + b + 1
                g.values[:, p] = -(100 * gi + b + 1)
    cm.state(2)[rc.state_slot] = torch.tensor([1.0, 2.0, 3.0])
    kept = cm.detach("a")
    cm.add("b")  # takes the state row that "a" had
    cm.state(2)[cm.requests["b"].state_slot] = 7.0
    with pytest.raises(OutOfPages, match="a copy of 70 kept tokens"):
        cm.fork(kept)  # group 0 has 4 pages left, five are needed
    assert [g.pool.n_free for g in cm.groups] == [4, 6]
    cm.truncate_kept(kept, 60)  # four blocks
    copy = cm.fork(kept)
    assert [g.pool.n_free for g in cm.groups] == [1, 5] and copy.length == 60  # a page each came back by the cut
    assert copy.blocks[1][:2] == [-1, -1] and not set(copy.blocks[0]) & set(kept.blocks[0])
    cm.drop(kept)  # the original goes; the copy stands alone
    rc = cm.attach("c", copy)
    for gi, g in enumerate(cm.groups):
        for b, p in enumerate(rc.blocks[gi]):
            if p >= 0:
                assert (g.keys[:, p] == 100 * gi + b + 1).all() and (g.values[:, p] == -(100 * gi + b + 1)).all()
    assert cm.state(2)[rc.state_slot].tolist() == [1.0, 2.0, 3.0]
    cm.set_state("c")
    assert cm.state(2)[rc.state_slot].tolist() == [0.0, 0.0, 0.0]
    cm.set_state("c", {2: torch.tensor([4.0, 5.0, 6.0])})
    assert cm.state(2)[rc.state_slot].tolist() == [4.0, 5.0, 6.0]
    cm.check()
    cm.release_all()
    assert [g.pool.n_free for g in cm.groups] == [9, 9] and not cm.kept


def test_kept_pages_go_to_a_file_and_into_another_pool(tmp_path):
    """``read_kept`` gathers the tokens' keys, values and state out of the pages, ``write_kept`` fills
    pages of another pool with them (another page size, scrambled pages); through a file with
    ``save_prompt_cache`` / ``load_prompt_cache`` (mlx_lm/models/cache.py:43-85, with the metadata
    that mlx_lm/cache_prompt.py:150-153 writes)."""
    import torch

    from mlx_lm_amd.prompt_cache import PromptCache, load_prompt_cache, save_prompt_cache, trim_prompt_cache

    needs = [CacheNeed(2, 16, 0), CacheNeed(1, 16, 0, v_head_dim=32), StateNeed((3,))]

    class Shim:  # what a PromptCache asks of an engine, over a pool on the CPU
        def __init__(self, page_size, n_pages):
            self.cache = CacheManager(needs, page_size, n_pages, 3, dtype=torch.float32, device="cpu")
            for name in ("read_kept", "write_kept", "attach", "detach", "add", "drop"):
                setattr(self, {"attach": "attach_request", "detach": "detach_request", "add": "add_request",
                               "drop": "drop_kept"}.get(name, name), getattr(self.cache, name))

        def context_len(self, rid):
            return self.cache.requests[rid].length

    a = Shim(16, 9)
    a.cache.add("junk"), a.cache.reserve("junk", 20), a.cache.commit("junk", 20)  # so that pages are not 0, 1, 2 ...
    cache = PromptCache()
    cache.checkout(a, "r")
    a.cache.reserve("r", 45), a.cache.commit("r", 45)
    rc = a.cache.requests["r"]
    g = torch.Generator().manual_seed(0)
    want = {}
    for slot in (0, 1):
        gi, i = a.cache.slot_group[slot]
        grp = a.cache.groups[gi]
        k = torch.randn(45, grp.need.n_kv_heads, grp.need.head_dim, generator=g)
        v = torch.randn(45, grp.need.n_kv_heads, grp.need.value_dim, generator=g)
        want[slot] = (k, v)
        for t in range(45):
            page = rc.blocks[gi][t // 16]
            grp.keys[i][page, :, t % 16] = k[t]
            grp.values[i][page, :, t % 16] = v[t]
    a.cache.state(2)[rc.state_slot] = torch.tensor([1.0, 2.0, 3.0])
    cache.checkin(a, "r")
    length, per_slot, state = cache.tensors()
    assert length == 45 and state[2].tolist() == [1.0, 2.0, 3.0]
    assert all(torch.equal(per_slot[s][0], want[s][0]) and torch.equal(per_slot[s][1], want[s][1]) for s in want)
    path = str(tmp_path / "cache.safetensors")
    save_prompt_cache(path, cache, {"model": "somewhere", "tokenizer_config": "{}"})
    loaded, metadata = load_prompt_cache(path, return_metadata=True)
    assert metadata == {"model": "somewhere", "tokenizer_config": "{}"}
    assert loaded.offset == 45 and loaded.engine is None and not loaded.is_trimmable()  # (it has state)
    assert trim_prompt_cache(loaded, 5) == 0
    # into a pool with pages of 32 tokens
    b = Shim(32, 4)
    loaded.checkout(b, "x")
    rb = b.cache.requests["x"]
    assert rb.length == 45 and b.cache.state(2)[rb.state_slot].tolist() == [1.0, 2.0, 3.0]
    for slot in (0, 1):
        gi, i = b.cache.slot_group[slot]
        grp = b.cache.groups[gi]
        for t in (0, 15, 16, 31, 32, 44):
            page = rb.blocks[gi][t // 32]
            assert torch.equal(grp.keys[i][page, :, t % 32], want[slot][0][t])
            assert torch.equal(grp.values[i][page, :, t % 32], want[slot][1][t])
    loaded.checkin(b, "x")
    b.cache.check()
    # a pool that is too small, and a model with other sizes
    again = load_prompt_cache(path)
    with pytest.raises(OutOfPages, match="a cache of 45 tokens"):
        again.checkout(Shim(16, 2), "y")
    assert not again.in_use or True
    other = Shim(16, 9)
    other.cache = CacheManager([CacheNeed(2, 16, 0), CacheNeed(1, 32, 0), StateNeed((3,))], 16, 9, 3,
                               dtype=torch.float32, device="cpu")
    other.write_kept = other.cache.write_kept
    with pytest.raises(ValueError, match="cache slot 1: keys"):
        load_prompt_cache(path).checkout(other, "z")
    # no request slot free: the cache stays as it was and can be used later
    full = Shim(16, 9)
    held = load_prompt_cache(path)
    for name in ("p", "q", "r"):
        full.cache.add(name)
    from mlx_lm_amd.cache import OutOfSlots

    with pytest.raises(OutOfSlots):
        held.checkout(full, "s")
    assert not held.in_use and held.offset == 45
    full.cache.release("p")
    held.checkout(full, "s")
    assert held.in_use and full.cache.requests["s"].length == 45
    held.checkin(full, "s")
    fresh = PromptCache()
    full.cache.add("p")
    with pytest.raises(OutOfSlots):
        fresh.checkout(full, "t")
    assert not fresh.in_use
    # an empty cache goes through a file as well
    save_prompt_cache(path, PromptCache())
    assert load_prompt_cache(path).offset == 0
