"""Generation through the entry points: greedy equals the plain implementation,
batches equal single requests, options mean what the reference's mean."""

import os
import subprocess
import sys

import pytest
import torch

import helpers
import plain_gpt2 as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def tiny(tmp_path_factory):
    out = {}
    for name in ("A", "B"):
        d = str(tmp_path_factory.mktemp(f"gen{name}"))
        config, weights = helpers.make_folder(d, name, 0.0)
        out[name] = (d, config, weights)
    return out


@pytest.fixture(scope="module")
def model_b(tiny):
    from mlx_lm_amd import load

    model, tok = load(tiny["B"][0], dtype="float32")
    assert tok is None
    return model


def _single(model, prompt, **kw):
    from mlx_lm_amd import stream_generate

    return [r.token for r in stream_generate(model, None, prompt, **kw)]


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_equals_plain(tiny, name):
    from mlx_lm_amd import generate, load, stream_generate

    d, config, weights = tiny[name]
    model, tok = load(d, dtype="float32")
    prompt = helpers.random_tokens(19, config["vocab_size"], seed=8)
    want = plain.greedy_generate(weights, config, prompt, 12)
    responses = list(stream_generate(model, tok, prompt, max_tokens=12, prefill_step_size=7))
    assert [r.token for r in responses] == want
    assert len(responses) == 12 and responses[-1].finish_reason == "length"
    assert all(r.finish_reason is None for r in responses[:-1])
    assert responses[-1].prompt_tokens == 19 and responses[-1].generation_tokens == 12
    lp = responses[0].logprobs
    want_lp = plain.log_softmax(plain.forward(weights, config, prompt)[-1])
    assert lp.shape == (config["vocab_size"],) and (lp.double().cpu() - want_lp).abs().max() < 1e-4
    assert generate(model, tok, prompt, max_tokens=12) == " ".join(str(t) for t in want)
    # bfloat16 agrees on nearly every token
    model16, _ = load(d, dtype="bfloat16")
    got16 = [r.token for r in stream_generate(model16, None, prompt, max_tokens=12)]
    assert sum(a == b for a, b in zip(got16, want)) >= 10


def test_max_tokens_logit_bias_and_stop(model_b, tiny):
    from mlx_lm_amd import make_logits_processors, stream_generate
    from mlx_lm_amd.generate import IdTokenizer

    prompt = [5, 6, 7]
    # mlx_lm tests/test_generate.py:37-64
    procs = make_logits_processors(logit_bias={0: 2000.0})
    assert _single(model_b, prompt, max_tokens=5, logits_processors=procs) == [0] * 5
    assert len(list(stream_generate(model_b, None, prompt, max_tokens=4))) == 4
    free = _single(model_b, prompt, max_tokens=6)
    tok = IdTokenizer()
    tok.add_eos_token(free[2])
    out = list(stream_generate(model_b, tok, prompt, max_tokens=6))
    stop_at = free.index(free[2])
    assert out[-1].finish_reason == "stop" and [r.token for r in out[:-1]] == free[:stop_at]
    with pytest.raises(ValueError, match="must be provided"):
        _single(model_b, [], max_tokens=1)
    with pytest.raises(ValueError, match="not supported"):
        _single(model_b, prompt, max_tokens=1, kv_bits=4)


def test_penalties_change_generation_as_the_plain_processors_do(model_b, tiny):
    from mlx_lm_amd import make_logits_processors

    _, config, weights = tiny["B"]
    prompt = helpers.random_tokens(10, config["vocab_size"], seed=3)
    procs = make_logits_processors(repetition_penalty=1.8, repetition_context_size=6,
                                   presence_penalty=0.7, frequency_penalty=0.4, frequency_context_size=4)
    got = _single(model_b, prompt, max_tokens=8, logits_processors=procs)
    seq, want = list(prompt), []
    for _ in range(8):
        x = plain.forward(weights, config, seq)[-1]
        x = plain.repetition_penalty(x, seq, 1.8, 6)
        x = plain.presence_penalty(x, seq, 0.7, 20)
        x = plain.frequency_penalty(x, seq, 0.4, 4)
        want.append(int(x.argmax()))
        seq.append(want[-1])
    assert got == want


def test_batches_equal_single_requests(model_b, tiny):
    """Greedy tokens do not depend on batch size, budget or pool size (incl. pre-emption);
    cf. mlx_lm tests/test_generate.py:182-310."""
    from mlx_lm_amd import batch_generate
    from mlx_lm_amd.engine import Engine
    from mlx_lm_amd.generate import BatchGenerator

    _, config, _ = tiny["B"]
    V = config["vocab_size"]
    prompts = [helpers.random_tokens(n, V, seed=n) for n in (7, 33, 90, 3, 50)]
    max_tokens = [2, 3, 24, 5, 17]
    single = [_single(model_b, p, max_tokens=m) for p, m in zip(prompts, max_tokens)]
    res = batch_generate(model_b, None, prompts, max_tokens=max_tokens, return_token_ids=True,
                         return_logprobs=True)
    assert res.token_ids == single
    assert res.stats.generation_tokens == sum(max_tokens) and res.stats.prompt_tokens == sum(map(len, prompts))
    assert all(len(l) == m and max(l) <= 0 for l, m in zip(res.logprobs, max_tokens))
    res = batch_generate(model_b, None, prompts, max_tokens=max_tokens, return_token_ids=True,
                         completion_batch_size=3, prefill_batch_size=2, prefill_step_size=8)
    assert res.token_ids == single
    # a pool of 12 pages: requests wait for pages and the growing ones get pre-empted
    small = Engine(model_b, dtype="float32", page_size=16, n_pages=12, max_requests=8)
    gen = BatchGenerator(model_b, engine=small, prefill_step_size=16, completion_batch_size=4)
    uids = gen.insert(prompts, max_tokens)
    got = {u: [] for u in uids}
    while responses := gen.next_generated():
        for r in responses:
            got[r.uid].append(r.token)
    assert [got[u] for u in uids] == single
    small.cache.check()
    assert small.cache.free_pages() == 12


def test_per_request_samplers_seeds_and_stops(model_b, tiny):
    from mlx_lm_amd import make_sampler
    from mlx_lm_amd.generate import BatchGenerator

    _, config, _ = tiny["B"]
    V = config["vocab_size"]
    prompts = [helpers.random_tokens(n, V, seed=40 + n) for n in (5, 21, 64)]
    samplers = [make_sampler(temp=0.8), make_sampler(temp=1.3, top_k=20), make_sampler(temp=0.9, top_p=0.8, min_p=0.01)]
    seeds = [11, 22, 33]

    def run(order, **kw):
        gen = BatchGenerator(model_b, max_tokens=10, **kw)
        uids = gen.insert([prompts[i] for i in order], samplers=[samplers[i] for i in order],
                          seeds=[seeds[i] for i in order])
        got = {u: [] for u in uids}
        while responses := gen.next_generated():
            for r in responses:
                got[r.uid].append(r.token)
        return {i: got[u] for i, u in zip(order, uids)}

    together = run([0, 1, 2])
    assert all(len(v) == 10 for v in together.values())
    # alone, in another order and under a tight budget: the same tokens
    assert run([1]) [1] == together[1]
    assert run([2, 0, 1], prefill_step_size=4, prefill_batch_size=1, completion_batch_size=2) == together
    other_seed = BatchGenerator(model_b, max_tokens=10)
    u = other_seed.insert([prompts[0]], samplers=[samplers[0]], seeds=[12])
    toks = []
    while responses := other_seed.next_generated():
        toks += [r.token for r in responses]
    assert toks != together[0]
    # per-request stop sequences (mlx_lm tests/test_generate.py:473-503)
    gen = BatchGenerator(model_b, max_tokens=10)
    greedy = _single(model_b, prompts[1], max_tokens=10)
    uids = gen.insert([prompts[1], prompts[1]], stop_matchers=[[greedy[3:5]], None])
    out = {u: [] for u in uids}
    while responses := gen.next_generated():
        for r in responses:
            out[r.uid].append((r.token, r.finish_reason))
    first_stop = next(i for i in range(1, 10) if greedy[i - 1 : i + 1] == greedy[3:5])
    assert out[uids[0]][-1] == (greedy[first_stop], "stop") and len(out[uids[0]]) == first_stop + 1
    assert out[uids[1]][-1] == (greedy[9], "length")


def test_custom_sampler_callable_and_remove(model_b):
    from mlx_lm_amd.generate import BatchGenerator

    fixed = lambda logprobs: torch.tensor([7])  # mlx_lm tests/test_generate.py:362-403
    assert _single(model_b, [1, 2, 3], max_tokens=3, sampler=fixed) == [7, 7, 7]
    gen = BatchGenerator(model_b, max_tokens=50, prefill_step_size=8)
    uids = gen.insert([list(range(1, 40)), [4, 5]])
    gen.next()
    gen.remove([uids[0]])  # mid-prompt
    got = []
    while responses := gen.next_generated():
        got += [r.uid for r in responses]
    assert set(got) == {uids[1]} and gen.engine.cache.free_pages() == gen.engine.cache.n_pages


def test_command_line(tiny):
    d, config, weights = tiny["A"]
    prompt = [3, 1, 4, 1, 5]
    want = plain.greedy_generate(weights, config, prompt, 6)
    env = dict(os.environ, PYTHONPATH=ROOT)
    out = subprocess.run(
        [sys.executable, "-m", "mlx_lm_amd", "generate", "--model", d, "--prompt-ids", "3,1,4,1,5",
         "--max-tokens", "6", "--dtype", "float32", "--verbose", "F"],
        capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert out.stdout.strip() == " ".join(map(str, want))
    out = subprocess.run(
        [sys.executable, "-m", "mlx_lm_amd", "generate", "--model", d, "--prompt", "3 1 4 1 5", "-m", "6",
         "--temp", "0.7", "--top-p", "0.9", "--seed", "3", "--dtype", "float32"],
        capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert "Prompt: 5 tokens" in out.stdout and "Generation: 6 tokens" in out.stdout and "Peak memory" in out.stdout


def test_many_interleaved_generators_keep_their_own_tokens(model_b, tiny):
    """Seven generators taken in turn, a token from each: every one's tokens (which stay on
    the device from its sampling call to its next step) equal those of the same request alone,
    however many other generators' sampling calls come in between."""
    from mlx_lm_amd import generate_step
    from mlx_lm_amd.sample_utils import make_sampler

    V = tiny["B"][1]["vocab_size"]
    sampler = make_sampler(temp=0.9)
    prompts = [helpers.random_tokens(5 + 3 * i, V, seed=400 + i) for i in range(7)]
    alone = [[t for t, _ in generate_step(p, model_b, max_tokens=10, sampler=sampler, seed=50 + i)]
             for i, p in enumerate(prompts)]
    assert len({tuple(a) for a in alone}) == 7  # the requests do differ
    gens = [generate_step(p, model_b, max_tokens=10, sampler=sampler, seed=50 + i) for i, p in enumerate(prompts)]
    together = [[] for _ in gens]
    for _ in range(10):
        for i, g in enumerate(gens):
            together[i].append(next(g)[0])
    for g in gens:
        g.close()
    assert together == alone


def test_two_batch_generators_and_a_generate_step_share_one_model(model_b, tiny):
    """Any number of generators may be live over one model (mlx_lm/generate.py:1596-1607,
    1712-1731: each ``BatchGenerator`` has caches and a uid counter of its own).  Here they share
    the model's engine and its pages: both generators number their requests from 0, are stepped
    in turn with a ``generate_step`` beside them, in a pool so small that requests wait or are
    pre-empted; every request makes the tokens it makes alone."""
    from mlx_lm_amd import generate_step
    from mlx_lm_amd.engine import Engine
    from mlx_lm_amd.generate import BatchGenerator

    V = tiny["B"][1]["vocab_size"]
    prompts_a = [helpers.random_tokens(n, V, seed=600 + n) for n in (40, 9, 23)]
    prompts_b = [helpers.random_tokens(n, V, seed=700 + n) for n in (31, 17)]
    prompt_c = helpers.random_tokens(12, V, seed=800)
    limits_a, limits_b, limit_c = [30, 20, 25], [28, 35], 22
    alone_a = [_single(model_b, p, max_tokens=m) for p, m in zip(prompts_a, limits_a)]
    alone_b = [_single(model_b, p, max_tokens=m) for p, m in zip(prompts_b, limits_b)]
    alone_c = _single(model_b, prompt_c, max_tokens=limit_c)
    # 14 pages of 16 tokens: what the five requests of the two generators grow to needs 18
    shared = Engine(model_b, dtype="float32", page_size=16, n_pages=14, max_requests=8)
    a = BatchGenerator(model_b, engine=shared, prefill_step_size=16, completion_batch_size=4)
    b = BatchGenerator(model_b, engine=shared, prefill_step_size=32, completion_batch_size=4)
    uids_a, uids_b = a.insert(prompts_a, limits_a), b.insert(prompts_b, limits_b)
    assert uids_a == [0, 1, 2] and uids_b == [0, 1]  # the same ids, and both live
    got_a, got_b, got_c = {u: [] for u in uids_a}, {u: [] for u in uids_b}, []
    c = generate_step(prompt_c, model_b, max_tokens=limit_c)  # on the model's own engine
    held_back = 0
    for _ in range(3000):
        live = False
        for gen, got in ((a, got_a), (b, got_b)):
            if not gen.scheduler.has_work:
                continue
            live = True
            try:
                _, responses = gen.next()
            except RuntimeError as e:  # the other generator holds every page just now
                assert "other generators" in str(e)
                held_back += 1
                continue
            for r in responses:
                got[r.uid].append(r.token)
        if len(got_c) < limit_c:
            live = True
            got_c.append(next(c)[0])
        if not live:
            break
        shared.cache.check()
    assert [got_a[u] for u in uids_a] == alone_a
    assert [got_b[u] for u in uids_b] == alone_b
    assert got_c == alone_c
    assert a.scheduler.stats.preemptions + b.scheduler.stats.preemptions + held_back > 0
    assert shared.cache.free_pages() == 14 and not shared.cache.requests
    # a generator that is dropped with requests live gives their pages back
    d = BatchGenerator(model_b, engine=shared, prefill_step_size=16)
    d.insert(prompts_a[:1], [50])
    d.next()
    assert shared.cache.requests
    d.close()
    assert shared.cache.free_pages() == 14 and not shared.cache.requests


def test_no_tokens_asked_for_none_made(model_b, tiny):
    """``max_tokens=0`` (mlx_lm/generate.py:448-461): nothing is yielded, and in a batch the
    request ends at once beside the others."""
    from mlx_lm_amd import batch_generate, generate_step

    V = tiny["B"][1]["vocab_size"]
    p = helpers.random_tokens(9, V, seed=3)
    assert list(generate_step(p, model_b, max_tokens=0)) == []
    out = batch_generate(model_b, None, [p, p], max_tokens=[0, 3], return_token_ids=True)
    assert out.token_ids[0] == [] and len(out.token_ids[1]) == 3


def test_penalty_histories_are_checked_against_the_vocabulary(model_b, tiny):
    from mlx_lm_amd.sample_utils import make_logits_processors

    V = tiny["B"][1]["vocab_size"]
    logits = torch.zeros(1, V, device="cuda")
    (proc,) = make_logits_processors(repetition_penalty=1.3)
    with pytest.raises(ValueError, match="vocabulary"):
        proc(torch.tensor([1, V + 5]), logits)
    proc(torch.tensor([1, V - 1]), logits)


def test_command_line_cache_geometry_and_random_weights(tiny, tmp_path):
    """The engine's own options: pages of 32 tokens in a pool of 8, a scheduler's limits, and
    weights drawn for a configuration instead of read (``--random-weights SEED --config FILE``:
    the same tokens as from the folder that the random-weights mode writes with that seed)."""
    import json

    from mlx_lm_amd.weights import write_model_folder

    d, config, weights = tiny["A"]
    prompt = [3, 1, 4, 1, 5]
    want = plain.greedy_generate(weights, config, prompt, 6)
    env = dict(os.environ, PYTHONPATH=ROOT)
    base = [sys.executable, "-m", "mlx_lm_amd", "generate", "--prompt-ids", "3,1,4,1,5", "--max-tokens", "6",
            "--dtype", "float32", "--verbose", "F"]
    out = subprocess.run(base + ["--model", d, "--block-size", "32", "--num-pages", "8", "--max-num-seqs", "2",
                                 "--max-num-batched-tokens", "3", "--prefill-step-size", "2"],
                         capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr[-2000:]
    assert out.stdout.strip() == " ".join(map(str, want))
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(helpers.TINY_B))
    folder = tmp_path / "drawn"
    write_model_folder(str(folder), dict(helpers.TINY_B), 12, "b")
    outs = []
    for source in (["--model", str(folder)], ["--random-weights", "12", "--config", str(cfg)]):
        out = subprocess.run(base + source, capture_output=True, text=True, env=env, timeout=300)
        assert out.returncode == 0, out.stderr[-2000:]
        outs.append(out.stdout.strip())
    assert outs[0] == outs[1] and len(outs[0].split()) == 6
    out = subprocess.run(base, capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode != 0 and "--model" in out.stderr
