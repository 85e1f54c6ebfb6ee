"""Going on from what an earlier request computed: ``prompt_cache`` of ``generate_step`` and
``stream_generate``, ``caches`` and ``return_prompt_caches`` of ``BatchGenerator`` and
``batch_generate``, ``trim_prompt_cache``.  Every continuation must give the tokens and the
log-probabilities of one uncached run over the same tokens, and of the plain implementation."""

import pytest
import torch

import helpers
import plain_gpt2 as plain

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def setup(request, tmp_path_factory):
    from mlx_lm_amd import load
    from mlx_lm_amd.engine import Engine

    d = str(tmp_path_factory.mktemp("pc"))
    config, weights = helpers.make_folder(d, "B", 0.0)
    model, _ = load(d, dtype=request.param)
    # pages of 16 tokens, so few that kept caches and live requests compete for them
    engine = Engine(model, dtype=request.param, page_size=16, n_pages=20, max_requests=8)
    return model, engine, config, weights, request.param


def _close(a, b, dtype):
    tol = 2e-4 if dtype == "float32" else 0.25
    return (a.double().cpu() - b.double().cpu()).abs().max().item() <= tol


def test_generate_step_goes_on_from_its_cache(setup):
    """mlx_lm tests/test_prompt_cache.py:184-204: two tokens with a cache, then the third from
    the second alone, are the tokens and logits of a run without a cache."""
    from mlx_lm_amd import generate_step, make_prompt_cache
    from mlx_lm_amd.generate import engine_for

    model, _, config, weights, dtype = setup
    prompt = helpers.random_tokens(21, config["vocab_size"], seed=3)
    toks, all_logits = zip(*generate_step(prompt, model, max_tokens=4))
    if dtype == "float32":
        assert list(toks) == plain.greedy_generate(weights, config, prompt, 4)
    cache = make_prompt_cache(model)
    i = 0
    for tok, logits in generate_step(prompt, model, prompt_cache=cache, max_tokens=2):
        assert tok == toks[i] and _close(logits, all_logits[i], dtype)
        i += 1
    assert i == 2 and cache.offset == 21 + 2 and not cache.in_use
    # the cache holds prompt, toks[0] and toks[1]: nothing to feed but a token that follows them
    for tok, logits in generate_step([toks[2]], model, prompt_cache=cache, max_tokens=1):
        assert tok == toks[3] and _close(logits, all_logits[3], dtype)
        i += 1
    assert i == 3 and cache.offset == 21 + 2 + 1 + 1
    pool = engine_for(model).cache
    assert pool.free_pages() == pool.n_pages - pool.blocks_for(cache.offset)
    cache.free()
    assert pool.free_pages() == pool.n_pages and cache.offset == 0
    pool.check()


def test_trim_takes_tokens_back(setup):
    """mlx_lm/models/cache.py:88-111; after a trim the next tokens are read at the earlier places."""
    from mlx_lm_amd import can_trim_prompt_cache, make_prompt_cache, stream_generate, trim_prompt_cache

    model, _, config, weights, dtype = setup
    V = config["vocab_size"]
    prompt = helpers.random_tokens(40, V, seed=5)
    other = helpers.random_tokens(9, V, seed=6)
    cache = make_prompt_cache(model)
    assert trim_prompt_cache(cache, 3) == 0  # nothing there yet
    list(stream_generate(model, None, prompt + [1, 2, 3], max_tokens=5, prompt_cache=cache))
    assert cache.offset == 48 and can_trim_prompt_cache(cache)
    assert trim_prompt_cache(cache, 8) == 8 and cache.offset == 40  # the prompt alone is left
    got = list(stream_generate(model, None, other, max_tokens=6, prompt_cache=cache))
    want = list(stream_generate(model, None, prompt + other, max_tokens=6))
    assert [r.token for r in got] == [r.token for r in want]
    assert all(_close(a.logprobs, b.logprobs, dtype) for a, b in zip(got, want))
    assert got[-1].prompt_tokens == 9  # only its own tokens were read
    if dtype == "float32":
        assert [r.token for r in want] == plain.greedy_generate(weights, config, prompt + other, 6)
    assert trim_prompt_cache(cache, 1000) == 40 + 9 + 6 and cache.offset == 0
    cache.free()


def test_a_generator_left_half_way_keeps_what_the_host_knows(setup):
    """A ``generate_step`` that is dropped after two tokens leaves prompt and those two tokens (the
    step in flight is forgotten); going on gives the uncached run's next tokens."""
    from mlx_lm_amd import generate_step, make_prompt_cache

    model, _, config, _, dtype = setup
    prompt = helpers.random_tokens(30, config["vocab_size"], seed=9)
    toks = [t for t, _ in generate_step(prompt, model, max_tokens=6)]
    cache = make_prompt_cache(model)
    g = generate_step(prompt, model, prompt_cache=cache, max_tokens=50)
    assert [next(g)[0], next(g)[0]] == toks[:2]
    g.close()
    assert not cache.in_use and cache.offset in (31, 32)  # toks[1] is known but perhaps not fed yet
    rest = [toks[1]] if cache.offset == 31 else []
    got = [t for t, _ in generate_step(rest + [toks[2]], model, prompt_cache=cache, max_tokens=3)]
    assert got == toks[3:6]
    cache.free()


def test_batch_generator_takes_caches_and_hands_them_back(setup):
    """mlx_lm tests/test_generate.py:590-640: the caches of a first round of requests go into a
    second round; its log-probabilities are those of single requests that go on from the same
    caches, which the batch left as they were."""
    from mlx_lm_amd import generate_step
    from mlx_lm_amd.generate import BatchGenerator

    model, engine, config, weights, dtype = setup
    V = config["vocab_size"]
    prompts_a = [helpers.random_tokens(n, V, seed=20 + n) for n in (5, 3, 18, 1)]
    prompts_b = [helpers.random_tokens(n, V, seed=40 + n) for n in (2, 7, 4, 17)]
    gen = BatchGenerator(model, engine=engine, max_tokens=10, prefill_batch_size=4, prefill_step_size=8,
                         completion_batch_size=2, return_prompt_caches=True)
    uids = gen.insert(prompts_a)
    caches, firsts = {}, {u: [] for u in uids}
    while responses := gen.next_generated():
        for r in responses:
            firsts[r.uid].append(r.token)
            if r.finish_reason is not None:
                caches[r.uid] = r.prompt_cache
    caches = [caches[u] for u in uids]
    assert [c.offset for c in caches] == [len(p) + 10 for p in prompts_a]
    held = sum(engine.cache.blocks_for(c.offset) for c in caches)
    assert engine.cache.free_pages() == 20 - held
    uids_b = gen.insert(prompts_b, caches=caches)
    batch = {u: [] for u in uids_b}
    second = {}
    while responses := gen.next_generated():
        for r in responses:
            batch[r.uid].append((r.token, r.logprobs))
            if r.finish_reason is not None:
                second[r.uid] = r.prompt_cache
        engine.cache.check()
    assert [c.offset for c in caches] == [len(p) + 10 for p in prompts_a]  # untouched
    for e, u in enumerate(uids_b):
        assert second[u].offset == caches[e].offset + len(prompts_b[e]) + 10
        second[u].free()
    for e, u in enumerate(uids_b):
        single = list(generate_step(prompts_b[e], model, max_tokens=10, prompt_cache=caches[e]))
        assert [t for t, _ in single] == [t for t, _ in batch[u]]
        assert all(_close(a[1], b[1], dtype) for a, b in zip(single, batch[u]))
        if dtype == "float32":  # and of the plain implementation over all the tokens in one sequence
            whole = prompts_a[e] + firsts[uids[e]] + prompts_b[e]
            assert [t for t, _ in single] == plain.greedy_generate(weights, config, whole, 10)
    for c in caches:
        c.free()
    assert engine.cache.free_pages() == 20 and not engine.cache.kept and not engine.cache.requests
    engine.cache.check()


def test_remove_hands_back_what_was_computed(setup):
    """mlx_lm/generate.py:1777-1802."""
    from mlx_lm_amd.generate import BatchGenerator, generate_step

    model, engine, config, _, dtype = setup
    V = config["vocab_size"]
    prompts = [helpers.random_tokens(n, V, seed=60 + n) for n in (37, 6)]
    alone = [t for t, _ in generate_step(prompts[0], model, max_tokens=8, engine=engine)]
    gen = BatchGenerator(model, engine=engine, max_tokens=40, prefill_step_size=16, prefill_batch_size=1)
    uids = gen.insert(prompts)
    gen.next()  # the first portion of the long prompt
    got = gen.remove([uids[0]], return_prompt_caches=True)
    cache = got[uids[0]]
    assert 0 < cache.offset < 37 and not cache.in_use
    gen.remove([uids[1]])
    assert engine.cache.free_pages() == 20 - engine.cache.blocks_for(cache.offset)
    rest = prompts[0][cache.offset:]
    assert [t for t, _ in generate_step(rest, model, max_tokens=8, prompt_cache=cache)] == alone
    cache.free()
    assert engine.cache.free_pages() == 20


def test_batch_generate_with_prompt_caches(setup):
    from mlx_lm_amd import batch_generate

    model, engine, config, _, dtype = setup
    V = config["vocab_size"]
    heads = [helpers.random_tokens(n, V, seed=80 + n) for n in (25, 11)]
    tails = [helpers.random_tokens(n, V, seed=90 + n) for n in (4, 9)]
    first = batch_generate(model, None, heads, max_tokens=1, return_prompt_caches=True, engine=engine)
    for c, h in zip(first.caches, heads):
        assert c.offset == len(h) + 1
        assert c.trim(1) == 1
    res = batch_generate(model, None, tails, prompt_caches=first.caches, max_tokens=7, return_token_ids=True,
                         engine=engine)
    want = batch_generate(model, None, [h + t for h, t in zip(heads, tails)], max_tokens=7,
                          return_token_ids=True, engine=engine)
    assert res.token_ids == want.token_ids and res.stats.prompt_tokens == 13
    for c in first.caches:
        c.free()
    assert engine.cache.free_pages() == 20 and not engine.cache.kept


def test_preemption_with_kept_caches_and_a_pool_that_they_fill(setup):
    """Requests on top of kept caches in a pool so small that the growing ones are pre-empted: they
    go back to their caches' tokens, read only their own again, and make the tokens they make alone.
    A cache that would not fit is refused with the pages named."""
    from mlx_lm_amd.cache import OutOfPages
    from mlx_lm_amd.generate import BatchGenerator, generate_step

    model, engine, config, _, dtype = setup
    V = config["vocab_size"]
    heads = [helpers.random_tokens(n, V, seed=100 + n) for n in (40, 33)]
    tails = [helpers.random_tokens(n, V, seed=110 + n) for n in (6, 20)]
    limits = [75, 70]
    alone = [[t for t, _ in generate_step(h + t, model, max_tokens=m, engine=engine)]
             for h, t, m in zip(heads, tails, limits)]
    gen = BatchGenerator(model, engine=engine, max_tokens=1, return_prompt_caches=True)
    uids = gen.insert(heads)
    caches = {}
    while responses := gen.next_generated():
        for r in responses:
            caches[r.uid] = r.prompt_cache
    caches = [caches[u] for u in uids]
    for c in caches:
        c.trim(1)
    # 20 pages: the two caches hold 3 + 3, their copies 6 more; 40+6+75 and 33+20+70 tokens need 8 + 8
    gen2 = BatchGenerator(model, engine=engine, prefill_step_size=16, completion_batch_size=4)
    uids2 = gen2.insert(tails, limits, caches=caches)
    got = {u: [] for u in uids2}
    while responses := gen2.next_generated():
        for r in responses:
            got[r.uid].append(r.token)
            if r.finish_reason is not None:
                r.prompt_cache.free()
        engine.cache.check()
    assert [got[u] for u in uids2] == alone
    assert gen2.scheduler.stats.preemptions > 0
    with pytest.raises(OutOfPages, match="a copy of"):
        [c.copy() for c in caches for _ in range(4)]
    import gc

    gc.collect()  # the copies that were made before the pool ran out go back with their objects
    for c in caches:
        c.free()
    assert engine.cache.free_pages() == 20 and not engine.cache.kept


def test_a_cache_goes_through_a_file_and_into_another_engine(setup, tmp_path):
    """``save_prompt_cache`` / ``load_prompt_cache`` (mlx_lm/models/cache.py:43-85; the reference's
    tests/test_prompt_cache.py:43-69 saves, loads and compares): the loaded cache gives the tokens
    of the one in memory, in the model's own engine and in one with pages of another size."""
    from mlx_lm_amd import generate_step, load_prompt_cache, make_prompt_cache, save_prompt_cache
    from mlx_lm_amd.engine import Engine

    model, engine, config, weights, dtype = setup
    V = config["vocab_size"]
    head = helpers.random_tokens(37, V, seed=130)
    tail = helpers.random_tokens(5, V, seed=131)
    want = [t for t, _ in generate_step(head + tail, model, max_tokens=9, engine=engine)]
    cache = make_prompt_cache(model)
    assert list(generate_step(head, model, max_tokens=0, prompt_cache=cache, engine=engine)) == []
    assert cache.offset == 37  # (no token asked for: the prompt is read into the cache, mlx_lm/cache_prompt.py:132-143)
    path = str(tmp_path / "c.safetensors")
    save_prompt_cache(path, cache, {"model": "m"})
    cache.free()
    assert engine.cache.free_pages() == 20
    loaded, meta = load_prompt_cache(path, return_metadata=True)
    assert meta == {"model": "m"} and loaded.offset == 37 and loaded.engine is None
    got = [t for t, _ in generate_step(tail, model, max_tokens=9, prompt_cache=loaded, engine=engine)]
    assert got == want and loaded.engine is engine and loaded.offset == 37 + 5 + 9
    # the token that ended that request has not gone through the model: it travels with the file
    assert loaded.pending == [want[-1]]
    more = helpers.random_tokens(3, V, seed=132)
    want_more = [t for t, _ in generate_step(head + tail + want + more, model, max_tokens=4, engine=engine)]
    path2 = str(tmp_path / "c2.safetensors")
    save_prompt_cache(path2, loaded)
    loaded.free()
    second = load_prompt_cache(path2)
    assert second.offset == 51 and second.pending == [want[-1]]
    assert [t for t, _ in generate_step(more, model, max_tokens=4, prompt_cache=second, engine=engine)] == want_more
    second.free()
    other = Engine(model, dtype=dtype, page_size=32, n_pages=6, max_requests=2)
    again = load_prompt_cache(path)
    assert [t for t, _ in generate_step(tail, model, max_tokens=9, prompt_cache=again, engine=other)] == want
    again.free()
    assert engine.cache.free_pages() == 20 and other.cache.free_pages() == 6


def test_cache_prompt_and_generate_on_the_command_line(tmp_path):
    """``cache_prompt`` writes the file that ``generate --prompt-cache-file`` goes on from, and the
    file names the model (mlx_lm/cache_prompt.py:150-153, mlx_lm/generate.py:2070-2096)."""
    import os
    import subprocess
    import sys

    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    d = str(tmp_path / "model")
    config, weights = helpers.make_folder(d, "A", 0.0)
    head, tail = [3, 1, 4, 1, 5, 9, 2, 6, 5, 3, 5, 8, 9, 7, 9, 3, 2, 3], [8, 4, 6]
    want = plain.greedy_generate(weights, config, head + tail, 6)
    env = dict(os.environ, PYTHONPATH=root)
    path = str(tmp_path / "head.safetensors")
    out = subprocess.run([sys.executable, "-m", "mlx_lm_amd", "cache_prompt", "--model", d, "--prompt-ids",
                          " ".join(map(str, head)), "--prompt-cache-file", path, "--dtype", "float32",
                          "--prefill-step-size", "7"], capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert "Processed     18 tokens" in out.stdout and "Saving..." in out.stdout
    out = subprocess.run([sys.executable, "-m", "mlx_lm_amd", "generate", "--prompt-cache-file", path, "--prompt-ids",
                          " ".join(map(str, tail)), "--max-tokens", "6", "--dtype", "float32", "--verbose", "F"],
                         capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert out.stdout.strip() == " ".join(map(str, want))


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_chains_of_requests_over_kept_caches(setup, seed):
    """Conversations of several turns in one generator over a pool that is too small for them all:
    each turn goes on from the cache that the turn before left (or from a copy that was cut back,
    or from one that went through ``remove`` half-way), requests are pre-empted, caches are freed
    at random.  In 32-bit every turn's tokens are those of one uncached request over all the
    conversation's tokens so far."""
    import random

    from mlx_lm_amd.generate import BatchGenerator, generate_step

    model, engine, config, _, dtype = setup
    if dtype != "float32":
        pytest.skip("token-for-token equality is a 32-bit matter")
    rng = random.Random(seed)
    V = config["vocab_size"]
    gen = BatchGenerator(model, engine=engine, prefill_step_size=16, prefill_batch_size=2, completion_batch_size=4,
                         return_prompt_caches=True)
    talks = []  # [tokens so far, cache or None]
    live = {}   # uid -> (talk index, tokens before this turn, prompt, limit)
    checked = turns = 0
    for _ in range(400):
        if len(live) < 5 and turns < 24 and rng.random() < 0.5:
            free_tokens = engine.cache.free_pages() * 16
            if talks and rng.random() < 0.6:
                i = rng.randrange(len(talks))
                if any(t[0] == i for t in live.values()) or talks[i][1] is None:
                    continue
            else:
                talks.append([[], None])
                i = len(talks) - 1
            so_far, cache = talks[i]
            prompt = helpers.random_tokens(rng.randint(1, 30), V, seed=rng.randrange(10**6))
            limit = rng.randint(1, 12)
            if len(so_far) + len(prompt) + limit > 150 or len(so_far) + len(prompt) + limit + 16 > free_tokens:
                continue
            if cache is not None and rng.random() < 0.3 and cache.offset > 3:  # cut the conversation back
                cut = rng.randint(1, 3)
                assert cache.trim(cut) == cut
                so_far = talks[i][0] = so_far[:-cut]
            uid = gen.insert([prompt], [limit], caches=[cache] if cache is not None else None)[0]
            live[uid] = (i, list(so_far), prompt, limit)
            turns += 1
        if not gen.scheduler.has_work:
            if turns >= 24 and not live:
                break
            continue
        if live and rng.random() < 0.04:  # taken out half-way: what it had computed goes on as the cache
            uid = rng.choice(list(live))
            i, before, prompt, limit = live.pop(uid)
            got = gen.remove([uid], return_prompt_caches=True)[uid]
            if talks[i][1] is not None:
                talks[i][1].free()
            known = before + prompt
            assert got.offset <= len(known) + limit
            # (the tokens that it had generated are not known here: go on from the prompt's part)
            keep = min(got.offset, len(known))
            got.trim(got.offset - keep)
            talks[i] = [known[:keep], got]
            continue
        _, responses = gen.next()
        for r in responses:
            if r.finish_reason is None:
                continue
            i, before, prompt, limit = live.pop(r.uid)
            made = r.all_tokens[len(prompt):]
            # (alone, on the model's own engine: the small pool is full of conversations)
            want = [t for t, _ in generate_step(before + prompt, model, max_tokens=limit)]
            assert made == want, (seed, r.uid)
            checked += 1
            if talks[i][1] is not None:
                talks[i][1].free()  # (the turn worked on a copy)
            talks[i] = [before + prompt + made, r.prompt_cache]
            assert r.prompt_cache.offset == len(talks[i][0])
            if rng.random() < 0.2:
                r.prompt_cache.free()
                talks[i][1] = None
        engine.cache.check()
    assert checked >= 8 and not live
    gen.close()
    for _, cache in talks:
        if cache is not None:
            cache.free()
    assert engine.cache.free_pages() == 20 and not engine.cache.kept and not engine.cache.requests


def test_a_batch_of_prompts_is_read_into_caches_without_a_token(setup):
    """``max_tokens=0`` with a cache in a ``BatchGenerator``: the prompts are read beside a request
    that decodes, each gives one response without a token that carries the cache, and a later
    request goes on from it."""
    from mlx_lm_amd import make_prompt_cache
    from mlx_lm_amd.generate import BatchGenerator, generate_step

    model, engine, config, _, dtype = setup
    V = config["vocab_size"]
    heads = [helpers.random_tokens(n, V, seed=150 + n) for n in (19, 40)]
    tail = helpers.random_tokens(4, V, seed=160)
    want = [[t for t, _ in generate_step(h + tail, model, max_tokens=5, engine=engine)] for h in heads]
    gen = BatchGenerator(model, engine=engine, prefill_step_size=16)
    uids = gen.insert(heads + [tail], [0, 0, 6], caches=[make_prompt_cache(model), make_prompt_cache(model), None])
    caches, tokens = {}, []
    while responses := gen.next_generated():
        for r in responses:
            if r.uid in uids[:2]:
                assert r.token is None and r.finish_reason == "length"
                caches[r.uid] = r.prompt_cache
            else:
                tokens.append(r.token)
    assert len(tokens) == 6 and [caches[u].offset for u in uids[:2]] == [19, 40]
    for u, w in zip(uids[:2], want):
        assert [t for t, _ in generate_step(tail, model, max_tokens=5, prompt_cache=caches[u])] == w
        caches[u].free()
    assert engine.cache.free_pages() == 20
