"""The scheduler's decisions with a stand-in engine (no GPU)."""

import random
from types import SimpleNamespace

import pytest

from mlx_lm_amd.cache import CacheManager
from mlx_lm_amd.config import CacheNeed
from mlx_lm_amd.engine.scheduler import Request, Scheduler, stops


class FakeEngine:
    """Keeps the real cache bookkeeping, runs no model; records what each step held."""

    def __init__(self, n_pages, max_positions=256, max_requests=8, page_size=16):
        self.cache = CacheManager([CacheNeed(2, 16, 0)], page_size, n_pages, max_requests)
        self.decoder = SimpleNamespace(max_positions=max_positions)
        self.log = []
        self.fed = 0

    def add_request(self, rid):
        return self.cache.add(rid)

    def end_request(self, rid):
        self.cache.release(rid)

    def has_request(self, rid):
        return rid in self.cache.requests

    def context_len(self, rid):
        return self.cache.requests[rid].length

    def truncate(self, rid, new_length):
        return self.cache.truncate(rid, new_length).length

    def detach_request(self, rid):
        return self.cache.detach(rid)

    def attach_request(self, rid, kept):
        return self.cache.attach(rid, kept)

    def drop_kept(self, kept):
        self.cache.drop(kept)

    def step(self, entries, fed=None):
        # the engine knows a request as (its scheduler's number, the scheduler's own id for it);
        # the log and the rows name it as its scheduler does
        for e in entries:
            self.cache.reserve(e.request_id, len(e.tokens))
            if e.fed_row >= 0:  # the token comes from the sampling call in flight: the right row of it
                assert fed is not None and fed[e.fed_row][0] == e.request_id[1] and len(e.tokens) == 1
                self.fed += 1
        rows = []
        for e in entries:
            start = self.cache.requests[e.request_id].length
            self.cache.commit(e.request_id, len(e.tokens))
            rows += [(e.request_id[1], start + w, tuple(e.tokens)) for w in e.want]
        self.log.append([(e.request_id[1], len(e.tokens), list(e.want)) for e in entries])
        self.cache.check()
        return rows


def token_for(rid, index):
    return (hash((rid, index)) % 997) + 1


def fake_sample(rows, requests):
    assert len(rows) == len(requests)
    out = []
    for (rid, pos, _), r in zip(rows, requests):
        assert rid == r.request_id and pos == r.offset + r.num_tokens - 1  # the row of the newest token
        out.append((token_for(rid, len(r.generated)), -1.0, None))
    return out


class TwoPhaseSample:
    """The same sampler in two phases, as the GPU's: ``launch`` returns at once, ``finish`` hands out
    the tokens; a scheduler given this overlaps its steps."""

    def launch(self, rows, requests):
        results = fake_sample(rows, requests)
        return SimpleNamespace(requests=list(requests), results=results, feedable=True,
                               tokens=[(r.request_id, t) for r, (t, _, _) in zip(requests, results)])

    def finish(self, job):
        return job.results

    def __call__(self, rows, requests):
        return self.finish(self.launch(rows, requests))


SAMPLERS = {"in turn": lambda: fake_sample, "overlapped": TwoPhaseSample}


def run_all(sched, limit=10000):
    done = {}
    for _ in range(limit):
        if not sched.has_work:
            return done
        for o in sched.step():
            done.setdefault(o.request_id, []).append(o)
    raise AssertionError("the scheduler did not finish")


def test_portions_under_a_token_budget_beside_decoding():
    eng = FakeEngine(n_pages=64)
    s = Scheduler(eng, fake_sample, max_num_seqs=4, max_num_batched_tokens=40, prefill_step_size=32)
    s.add(Request("a", list(range(1, 71)), 3))
    s.step()
    assert eng.log[-1] == [("a", 32, [])]
    s.add(Request("b", list(range(1, 11)), 5))
    s.step()  # a goes on with 32 more, b gets the 8 left of the budget
    assert eng.log[-1] == [("a", 32, []), ("b", 8, [])]
    outs = s.step()  # a's last 6 (sampled), b's last 2 (sampled)
    assert eng.log[-1] == [("a", 6, [5]), ("b", 2, [1])]
    assert [o.request_id for o in outs] == ["a", "b"] and outs[0].token == token_for("a", 0)
    s.add(Request("c", list(range(1, 60)), 2))
    s.step()  # decoding tokens first, then c's first portion in the same step
    assert eng.log[-1] == [("a", 1, [0]), ("b", 1, [0]), ("c", 32, [])]
    done = run_all(s)
    assert [o.finish_reason for o in done["c"]] == [None, "length"]
    assert eng.cache.free_pages() == 64 and not eng.cache.requests


@pytest.mark.parametrize("mode", SAMPLERS)
def test_max_tokens_stop_and_positions(mode):
    eng = FakeEngine(n_pages=64, max_positions=40)
    s = Scheduler(eng, SAMPLERS[mode]())
    for rid, n, mt in (("a", 5, 2), ("b", 7, 3), ("c", 3, 4), ("d", 9, 5)):
        s.add(Request(rid, list(range(1, n + 1)), mt))
    s.add(Request("stop", [1, 2, 3], 50, stop_sequences=[[token_for("stop", 1), token_for("stop", 2)]]))
    s.add(Request("long", list(range(1, 31)), 100))
    done = run_all(s)
    assert [len(done[r]) for r in "abcd"] == [2, 3, 4, 5]  # per-request max_tokens
    assert all(done[r][-1].finish_reason == "length" for r in "abcd")
    assert [o.finish_reason for o in done["stop"]] == [None, None, "stop"]  # the stopping token is reported
    assert len(done["long"]) == 40 - 30 and done["long"][-1].finish_reason == "length"
    # tokens are those of a request run alone, whatever shared its steps
    assert [o.token for o in done["d"]] == [token_for("d", i) for i in range(5)]
    assert stops([4, 5, 6], [[5, 6]]) and not stops([5, 6, 4], [[5, 6]]) and not stops([6], [[5, 6]])


@pytest.mark.parametrize("mode", SAMPLERS)
def test_admission_waits_for_pages_and_keeps_order(mode):
    eng = FakeEngine(n_pages=6)
    s = Scheduler(eng, SAMPLERS[mode](), max_num_seqs=8)
    s.add(Request("a", list(range(1, 50)), 4))  # 4 pages
    s.add(Request("b", list(range(1, 40)), 4))  # 3 pages: has to wait
    s.add(Request("c", [1, 2], 4))  # would fit, but b is first
    first = s.step()
    assert [r.request_id for r in s.running] == ["a"] and [r.request_id for r in s.waiting] == ["b", "c"]
    done = run_all(s)
    done["a"] = first + done["a"]
    assert sorted(done) == ["a", "b", "c"] and all(len(v) == 4 for v in done.values())
    first_step = {rid: next(i for i, st in enumerate(eng.log) if any(e[0] == rid for e in st)) for rid in "abc"}
    assert first_step["a"] < first_step["b"] <= first_step["c"]


@pytest.mark.parametrize("mode", SAMPLERS)
def test_preemption_when_pages_run_out(mode):
    eng = FakeEngine(n_pages=5, max_positions=200)
    s = Scheduler(eng, SAMPLERS[mode](), max_num_seqs=4)
    s.add(Request("old", list(range(1, 31)), 40))  # 2 pages, grows to 5
    s.add(Request("new", list(range(1, 17)), 40))  # 2 pages with its first token
    done = run_all(s)
    assert s.stats.preemptions >= 1
    pre = [r for r in ("old", "new")]
    assert len(done["old"]) == 40 and len(done["new"]) == 40
    # the pre-empted request went on where it was: same tokens as alone
    for rid in pre:
        assert [o.token for o in done[rid]] == [token_for(rid, i) for i in range(40)]
    # the newer request was the victim and re-read prompt + generated as one prompt
    reread = [st for st in eng.log if any(e[0] == "new" and e[1] > 16 for e in st)]
    assert reread
    assert eng.cache.free_pages() == 5


def test_what_cannot_fit_is_refused_at_once():
    eng = FakeEngine(n_pages=4, max_positions=100)
    s = Scheduler(eng, fake_sample)
    with pytest.raises(ValueError, match="cache holds"):
        s.add(Request("big", list(range(1, 60)), 30))
    with pytest.raises(ValueError, match="positions"):
        s.add(Request("long", list(range(1, 120)), 1))
    with pytest.raises(ValueError, match="at least one token"):
        s.add(Request("empty", [], 1))
    s.add(Request("ok", [1, 2, 3], 2))
    with pytest.raises(ValueError, match="in use"):
        s.add(Request("ok", [1], 1))


@pytest.mark.parametrize("mode", SAMPLERS)
def test_abort_frees_everything(mode):
    eng = FakeEngine(n_pages=16)
    s = Scheduler(eng, SAMPLERS[mode](), max_num_batched_tokens=16, prefill_step_size=16)
    s.add(Request("a", list(range(1, 60)), 5))
    s.add(Request("b", list(range(1, 20)), 5))
    s.step()
    s.abort("a")  # mid-prompt
    s.abort("b")  # still waiting or just admitted
    assert not s.has_work and eng.cache.free_pages() == 16
    with pytest.raises(KeyError):
        s.abort("a")


@pytest.mark.parametrize("mode", SAMPLERS)
@pytest.mark.parametrize("seed", range(5))
def test_random_load_every_request_finishes_with_its_own_tokens(seed, mode):
    rng = random.Random(seed)
    P = 128
    eng = FakeEngine(n_pages=rng.choice([8, 12, 30]), max_positions=P, max_requests=6)
    s = Scheduler(eng, SAMPLERS[mode](), max_num_seqs=rng.choice([2, 4, 6]),
                  max_num_batched_tokens=rng.choice([8, 33, 256]), prefill_step_size=rng.choice([5, 64]))
    want, done, added = {}, {}, 0
    for _ in range(3000):
        if added < 25 and rng.random() < 0.3:
            n, mt = rng.randint(1, 100), rng.randint(1, 40)
            rid = f"r{added}"
            s.add(Request(rid, [rng.randint(1, 900) for _ in range(n)], mt))
            want[rid] = min(mt, max(1, P - n))
            added += 1
        if s.has_work:
            for o in s.step():
                done.setdefault(o.request_id, []).append(o)
        elif added == 25:
            break
        assert len(s.running) <= s.max_num_seqs
        assert all(sum(e[1] for e in st) <= s.max_num_batched_tokens for st in eng.log[-1:])
    assert sorted(done) == sorted(want)
    for rid, outs in done.items():
        assert len(outs) == want[rid], rid
        assert [o.token for o in outs] == [token_for(rid, i) for i in range(len(outs))]
        assert outs[-1].finish_reason == "length" and all(o.finish_reason is None for o in outs[:-1])
    assert eng.cache.free_pages() == eng.cache.n_pages
    assert (eng.fed > 0) == (mode == "overlapped")


def test_overlapped_steps_what_is_known_early_and_what_is_found_late():
    """Steps overlap: a step is launched while the tokens of the one before are still on the device.
    A request whose token in flight is its last (max_tokens) is left out of that step; a stop
    sequence is only seen when the token is read, so the request takes part in one step too many,
    whose token is dropped; outputs come a step late."""
    eng = FakeEngine(n_pages=64)
    s = Scheduler(eng, TwoPhaseSample(), max_num_seqs=4)
    s.add(Request("len", [1, 2, 3], 2))
    s.add(Request("stop", [4, 5], 50, stop_sequences=[[token_for("stop", 1)]]))
    s.add(Request("on", [6], 6))
    assert s.step() == []  # the prompts run, sampling is in flight
    assert eng.log[-1] == [("len", 3, [2]), ("stop", 2, [1]), ("on", 1, [0])]
    outs = s.step()  # launches the first decode step, then reads the first tokens
    assert eng.log[-1] == [("len", 1, [0]), ("stop", 1, [0]), ("on", 1, [0])] and eng.fed == 3
    assert [(o.request_id, o.token, o.finish_reason) for o in outs] == [
        (r, token_for(r, 0), None) for r in ("len", "stop", "on")]
    outs = s.step()  # "len" is left out: its second token, in flight, is its last
    assert eng.log[-1] == [("stop", 1, [0]), ("on", 1, [0])]
    assert [(o.request_id, o.finish_reason) for o in outs] == [("len", "length"), ("stop", "stop"), ("on", None)]
    assert [r.request_id for r in s.running] == ["on"]  # "stop" is gone, though it was in the step just launched
    outs = s.step()
    assert eng.log[-1] == [("on", 1, [0])]
    assert [(o.request_id, o.token) for o in outs] == [("on", token_for("on", 2))]  # the token too many is dropped
    done = run_all(s)
    assert [o.token for o in done["on"]] == [token_for("on", i) for i in range(3, 6)]
    assert done["on"][-1].finish_reason == "length"
    assert eng.cache.free_pages() == 64 and not eng.cache.requests and not s.has_work


def test_overlapped_steps_abort_and_preemption_with_a_token_in_flight():
    eng = FakeEngine(n_pages=16)
    s = Scheduler(eng, TwoPhaseSample(), max_num_seqs=4)
    s.add(Request("a", [1, 2, 3], 10))
    s.add(Request("b", [4, 5, 6], 10))
    s.step()
    s.step()
    s.abort("a")  # its token is in flight: dropped when it is read
    outs = s.step()
    assert [o.request_id for o in outs] == ["b"]
    done = run_all(s)
    assert [o.token for o in outs + done["b"]] == [token_for("b", i) for i in range(1, 10)]
    assert eng.cache.free_pages() == 16
    # pre-emption of a request whose token is in flight: the token is kept, the request waits a
    # step and then reads prompt and generated tokens as one prompt
    eng = FakeEngine(n_pages=5, max_positions=200)
    s = Scheduler(eng, TwoPhaseSample(), max_num_seqs=4)
    s.add(Request("old", list(range(1, 31)), 40))
    s.add(Request("new", list(range(1, 17)), 40))
    done = run_all(s)
    assert s.stats.preemptions >= 1
    for rid in ("old", "new"):
        assert [o.token for o in done[rid]] == [token_for(rid, i) for i in range(40)]
    assert eng.cache.free_pages() == 5


@pytest.mark.parametrize("mode", list(SAMPLERS))
def test_a_request_for_no_tokens_is_over_at_once(mode):
    """``max_tokens=0``: no step, no sampled token (mlx_lm/generate.py:448-461 yields nothing)."""
    eng = FakeEngine(n_pages=16)
    sched = Scheduler(eng, SAMPLERS[mode](), max_num_seqs=4)
    r = sched.add(Request("none", [1, 2, 3], 0))
    assert r.finish_reason == "length" and not sched.has_work and not r.live
    sched.add(Request("one", [4, 5], 1))
    done = run_all(sched)
    assert list(done) == ["one"] and r.generated == [] and not eng.cache.requests
    assert all(rid != "none" for step in eng.log for rid, _, _ in step)


@pytest.mark.parametrize("mode", SAMPLERS)
def test_two_schedulers_share_an_engine_with_the_same_request_ids(mode):
    """Any number of generators may be live over one model, each numbering its requests from 0
    (mlx_lm/generate.py:1596-1607,1712-1731): the engine keeps them apart, a scheduler that finds
    the last slot or the pages taken leaves its request waiting (not lost), and each request makes
    the tokens it makes alone."""
    eng = FakeEngine(n_pages=7, max_positions=200, max_requests=3)
    a = Scheduler(eng, SAMPLERS[mode](), max_num_seqs=4)
    b = Scheduler(eng, SAMPLERS[mode](), max_num_seqs=4)
    for s in (a, b):
        s.add(Request(0, list(range(1, 31)), 30))  # 2 pages, grows to 4
        s.add(Request(1, list(range(1, 10)), 20))  # 1 page, grows to 2
    done = {id(a): {}, id(b): {}}
    held_back = False
    for _ in range(2000):
        if not (a.has_work or b.has_work):
            break
        for s in (a, b):
            if not s.has_work:
                continue
            try:
                outs = s.step()
            except RuntimeError as e:  # the other scheduler holds everything: said so, nothing lost
                assert "other generators" in str(e)
                assert len(s.waiting) + len(s.running) > 0
                held_back = True
                continue
            for o in outs:
                done[id(s)].setdefault(o.request_id, []).append(o.token)
        eng.cache.check()
    assert not (a.has_work or b.has_work)
    for s in (a, b):
        assert done[id(s)] == {0: [token_for(0, i) for i in range(30)], 1: [token_for(1, i) for i in range(20)]}
    assert a.stats.preemptions + b.stats.preemptions >= 1 or held_back
    assert eng.cache.free_pages() == 7 and not eng.cache.requests


def test_admission_that_fails_keeps_the_request_first_in_line():
    eng = FakeEngine(n_pages=16, max_requests=1)
    a = Scheduler(eng, fake_sample)
    b = Scheduler(eng, fake_sample)
    a.add(Request("x", [1, 2, 3], 3))
    a.step()  # takes the only slot
    rb = b.add(Request("x", [4, 5], 2))
    with pytest.raises(RuntimeError, match="1 requests of other generators"):
        b.step()
    assert list(b.waiting) == [rb] and rb.live and not b.running
    run_all(a)
    done = run_all(b)
    assert [o.token for o in done["x"]] == [token_for("x", 0), token_for("x", 1)]
    # a scheduler that is closed gives back what its requests hold
    a.add(Request("y", list(range(1, 40)), 5))
    a.step()
    assert eng.cache.requests
    a.close()
    assert not eng.cache.requests and eng.cache.free_pages() == 16 and not a.has_work


@pytest.mark.parametrize("mode", SAMPLERS)
def test_a_request_goes_on_from_a_kept_cache_and_leaves_its_tokens_there(mode):
    """``generate_step(..., prompt_cache=c)`` of the reference updates the cache in place: after
    the call it holds the prompt and every generated token, the last one too
    (mlx_lm/generate.py:306,329-331,444-461; tests/test_prompt_cache.py:184-204), and the next
    call reads only its own tokens on top.  Here the request's pages simply stay held."""
    from mlx_lm_amd.prompt_cache import PromptCache, can_trim_prompt_cache, trim_prompt_cache

    eng = FakeEngine(n_pages=8, max_positions=64)
    c = PromptCache()
    s = Scheduler(eng, SAMPLERS[mode]())
    prompt = list(range(1, 21))
    s.add(Request("a", prompt, 3, kept=c))
    done = run_all(s)
    first = [o.token for o in done["a"]]
    assert first == [token_for("a", i) for i in range(3)]
    assert c.offset == 23 and not c.in_use and not eng.cache.requests  # prompt and all three tokens
    # the token that ended the request has not gone through the model: the cache keeps it for the
    # next request to read first
    assert c.pending == [first[-1]] and eng.cache.kept[0].length == 22
    assert eng.cache.free_pages() == 8 - 2 and len(eng.cache.kept) == 1
    eng.cache.check()
    # the next request brings one token and starts at position 23
    s2 = Scheduler(eng, SAMPLERS[mode]())
    r = s2.add(Request("a", [777], 2, kept=c))
    assert r.offset == 22 and r.prefix == [first[-1]] and c.offset == 23 and c.claimed
    with pytest.raises(ValueError, match="in use"):  # a cache serves one request at a time
        s2.add(Request("b", [5], 1, kept=c))
    before = len(eng.log)
    early = s2.step()
    done = run_all(s2)
    assert eng.log[before] == [("a", 2, [1])]  # the pending token and its own, nothing else
    assert c.offset == 23 + 1 + 2 and len(early) + len(done["a"]) == 2 and not c.claimed
    # what does not fit the positions on top of the cache is refused
    with pytest.raises(ValueError, match="on top of the 26 of its cache"):
        Scheduler(eng, fake_sample).add(Request("x", list(range(1, 60)), 1, kept=c))
    # a cache goes on only in the engine whose pool holds it
    with pytest.raises(ValueError, match="another engine"):
        Scheduler(FakeEngine(n_pages=8, max_positions=64), fake_sample).add(Request("y", [1], 1, kept=c))
    # trimming, then giving the pages back
    assert can_trim_prompt_cache(c) and trim_prompt_cache(c, 10) == 10 and c.offset == 16
    assert eng.cache.free_pages() == 8 - 1
    eng.cache.check()
    c.free()
    assert eng.cache.free_pages() == 8 and not eng.cache.kept and c.offset == 0


@pytest.mark.parametrize("mode", SAMPLERS)
def test_kept_caches_under_preemption_and_abort(mode):
    from mlx_lm_amd.prompt_cache import PromptCache

    eng = FakeEngine(n_pages=6, max_positions=200)
    c = PromptCache()
    s = Scheduler(eng, SAMPLERS[mode](), max_num_seqs=4)
    s.add(Request("seed", list(range(1, 18)), 1, kept=c))  # 17 + 1 tokens: two pages kept
    run_all(s)
    assert c.offset == 18
    # "old" grows until the pool is full; "new", on top of the kept cache, is the victim: it goes
    # back to the 18 tokens of its cache and reads only its own tokens again
    s.add(Request("old", list(range(1, 31)), 20))
    s.add(Request("new", list(range(1, 11)), 30, kept=c))
    done = run_all(s)
    assert s.stats.preemptions >= 1
    assert [o.token for o in done["new"]] == [token_for("new", i) for i in range(30)]
    assert [o.token for o in done["old"]] == [token_for("old", i) for i in range(20)]
    assert c.offset == 18 + 10 + 30 and eng.cache.free_pages() == 6 - 4
    reread = [e for st in eng.log for e in st if e[0] == "new" and e[1] > 10]
    assert reread and all(e[1] <= 10 + 30 for e in reread)  # never the cache's own 18 tokens
    eng.cache.check()
    # taken out half-way with an empty cache to keep what it computed
    s.add(Request("cut", list(range(1, 21)), 5))
    s.max_num_batched_tokens = s.prefill_step_size = 16
    s.step()
    half = PromptCache()
    s.abort("cut", keep=half)
    assert half.offset == 16 and not s.has_work
    half.free()
    c.free()
    assert eng.cache.free_pages() == 6 and not eng.cache.kept


@pytest.mark.parametrize("mode", SAMPLERS)
def test_no_tokens_asked_for_on_top_of_a_cache_reads_the_prompt_into_it(mode):
    """mlx_lm/cache_prompt.py:132-143 fills a cache with ``generate_step(..., max_tokens=0,
    prompt_cache=cache)``: the whole prompt is read, nothing is sampled."""
    from mlx_lm_amd.prompt_cache import PromptCache

    eng = FakeEngine(n_pages=8, max_positions=64)
    c = PromptCache()
    s = Scheduler(eng, SAMPLERS[mode](), prefill_step_size=8)
    r = s.add(Request("fill", list(range(1, 22)), 0, kept=c))
    assert r.fill_only and s.has_work
    assert run_all(s) == {}
    assert c.offset == 21 and not c.in_use and r.finish_reason == "length"
    assert [e[1] for st in eng.log for e in st] == [8, 8, 5] and all(e[2] == [] for st in eng.log for e in st)
    assert eng.cache.free_pages() == 8 - 2
    # without a cache there is nothing to do
    assert s.add(Request("none", [1, 2, 3], 0)).finish_reason == "length" and not s.has_work
    # beside a request that decodes
    s.add(Request("gen", [5, 6, 7], 4))
    s.add(Request("more", [9] * 10, 0, kept=c))
    done = run_all(s)
    assert list(done) == ["gen"] and len(done["gen"]) == 4 and c.offset == 31
    c.free()
    assert eng.cache.free_pages() == 8
    eng.cache.check()


def test_a_model_with_a_window_takes_no_prompt_cache():
    from mlx_lm_amd.config.plan import CacheNeed
    from mlx_lm_amd.prompt_cache import PromptCache

    eng = FakeEngine(n_pages=8, max_positions=64)
    eng.cache = CacheManager([CacheNeed(2, 16, 24)], 16, 8, 4)
    s = Scheduler(eng, fake_sample)
    with pytest.raises(ValueError, match="window"):
        s.add(Request("w", [1, 2, 3], 2, kept=PromptCache()))
    s.add(Request("w", [1, 2, 3], 2))  # without one it runs
    assert len(run_all(s)["w"]) == 2
