"""The engine at the layer sizes of the published GPT-2 models (random weights): logits against
the plain implementation and against the same request run whole, the replay program in portions
of fixed sizes, and continuous batching under load.

Widths, heads, inner sizes, vocabulary and positions are the real ones.  Where a test runs
fewer layers than the model has, it says so: ``n_layer`` is what runs, ``N_LAYER_FULL`` what
the model of that name has.  Every test takes seconds on the GPU.
"""

import json
import os
import random
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_gpt2 as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": 2e-5, "bfloat16": 2.5e-2}


def _gpt2(n_layer, n_embd, n_head):
    return dict(model_type="gpt2", n_layer=n_layer, n_embd=n_embd, n_head=n_head, n_inner=4 * n_embd,
                vocab_size=50257, n_positions=1024, n_ctx=1024, layer_norm_epsilon=1e-5,
                activation_function="gelu_new")


# name: (what the tests run, layers of the full model, seed of the weights)
N_LAYER_FULL = {"xl": 48, "xl4": 48, "large": 36, "small": 12}
# Spread of the attention scores where the weights are sharpened.  bfloat16 rounds queries, keys and
# the cache; the sharper the softmax, the more of that rounding reaches the logits: measured at
# these sizes, evenly over all 1,024 positions, 0.4 % of the largest logit unsharpened, 1.2 % at a
# spread of 3 and 3.5 % at 6 (float32: 1e-6 at every spread), so bfloat16 is tested at 3.
SHARP = {"xl4": {"float32": 6.0, "bfloat16": 3.0}}
SIZES = {
    "xl": (_gpt2(12, 1600, 25), 2),      # 12 of 48 layers
    "xl4": (_gpt2(4, 1600, 25), 7),      # 4 of 48 layers: every position against the plain implementation
    "large": (_gpt2(36, 1280, 20), 4),   # all 36
    "small": (_gpt2(12, 768, 12), 3),    # all 12
}


@pytest.fixture(scope="module")
def folder_for(tmp_path_factory):
    made = {}

    def get(name, dtype=None):
        sharp = SHARP.get(name, {}).get(dtype, 0.0)
        if (name, sharp) not in made:
            from mlx_lm_amd.weights import write_model_folder

            config, seed = SIZES[name]
            assert config["n_layer"] <= N_LAYER_FULL[name]
            d = str(tmp_path_factory.mktemp(name))
            write_model_folder(d, dict(config), seed, "b", dtype="float32")
            if sharp:
                # peaked attention: a key dropped among a thousand, or taken from a wrong page, shows
                from safetensors.torch import load_file, save_file

                f = os.path.join(d, "model.safetensors")
                save_file(helpers.sharpen({k: v.clone() for k, v in load_file(f).items()}, config, sharp), f)
            made[name, sharp] = d
        return made[name, sharp], SIZES[name][0]

    return get


def _plain_weights(folder, config, dtype):
    from safetensors.torch import load_file

    w = plain.from_checkpoint_layout(
        {k: v.float() for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}, config["n_layer"])
    return helpers.round_matrices_to_bf16(w) if dtype == "bfloat16" else w


def _err(got, want):
    return (got.double().cpu() - want.double().cpu()).abs().max().item()


def _run(engine, rid, tokens, cuts):
    from mlx_lm_amd.engine import StepEntry

    engine.add_request(rid)
    rows, i = [], 0
    for n in cuts:
        rows.append(engine.step([StepEntry(rid, tokens[i : i + n], list(range(n)))]).cpu())
        i += n
    assert i == len(tokens)
    engine.end_request(rid)
    return torch.cat(rows)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpt2_xl_sizes_whole_decoded_portions_and_mixed(folder_for, dtype):
    """Width 1600, 25 heads of 64, inner 6400, 50,257 tokens, 1,024 positions (12 of 48 layers):
    one request of 1,024 tokens whole, with its last 32 tokens one by one, and in portions of
    changing size, against the plain implementation on the first 128 positions and against the
    whole run everywhere; then four requests mixed with so few pages that they are used again."""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    folder, config = folder_for("xl")
    V, n = config["vocab_size"], 1024
    tokens = helpers.random_tokens(n, V, seed=2)
    weights = _plain_weights(folder, config, dtype)
    want = plain.forward(weights, config, tokens[:128])
    scale = want.abs().max().item()
    model, _ = load_model(folder, dtype=dtype)
    eng = Engine(model, dtype=dtype, page_size=16, n_pages=n // 16 + 4, max_requests=4)
    whole = _run(eng, "whole", tokens, [n])
    assert _err(whole[:128], want) <= TOL[dtype] * scale, "whole against the plain implementation"
    scale = whole.abs().max().item()
    decoded = _run(eng, "decoded", tokens, [n - 32] + [1] * 32)
    assert _err(decoded, whole) <= TOL[dtype] * scale, "last 32 one by one"
    portions = _run(eng, "portions", tokens, helpers.cuts_changing(n))
    assert _err(portions, whole) <= TOL[dtype] * scale, "portions of changing size"
    assert _err(portions[:128], want) <= TOL[dtype] * want.abs().max().item()
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages
    del eng

    lengths = [300, 130, 210, 64, 170, 90]
    seqs, steps = helpers.mixed_trace(config, seed=21, lengths=lengths)
    eng = Engine(model, dtype=dtype, page_size=16, n_pages=helpers.held(lengths, 4) // 16, max_requests=4)
    assert sum((m + 15) // 16 for m in lengths) > eng.cache.n_pages  # pages are used again
    got = {rid: [] for rid in seqs}
    for s in steps:
        for e in s["entries"]:
            if not eng.has_request(e["id"]):
                eng.add_request(e["id"])
        eng.cache.poison_free_pages()
        logits = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]]).cpu()
        i = 0
        for e in s["entries"]:
            got[e["id"]].append(logits[i : i + len(e["want"])])
            i += len(e["want"])
        for rid in s["end"]:
            eng.end_request(rid)
    eng.cache.check()
    assert any(len(s["entries"]) == 4 for s in steps)
    alone = Engine(model, dtype=dtype, page_size=16, n_pages=20, max_requests=2)
    for rid, toks in seqs.items():
        ref = _run(alone, rid, toks, [len(toks)])
        assert _err(torch.cat(got[rid]), ref) <= TOL[dtype] * ref.abs().max().item(), f"mixed, request {rid}"
        if rid == "r1":
            w = plain.forward(weights, config, toks)
            assert _err(ref, w) <= TOL[dtype] * w.abs().max().item(), "a mixed request against the plain implementation"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpt2_xl_widths_every_position_and_every_kind_of_step_against_the_plain_implementation(folder_for, dtype):
    """Width 1600, 25 heads of 64, inner 6400, 50,257 tokens, 1,024 positions, 4 of 48 layers.  The
    plain implementation runs the 1,024 tokens once (float64); every run of the engine is compared
    with *it*, not with another run of the engine: at all 1,024 positions on 768 columns of the
    vocabulary, and on the whole vocabulary at 72 positions (among them 0, 127 to 129 -- the edge of
    the prefill kernel's tile of queries -- 511 to 513 and 1,023).  Runs: the request whole; its
    last 32 tokens one by one (contexts 992 to 1,023); portions of changing size down to two
    tokens; and single decode steps of 64, 40 and 12 requests whose contexts are spread over 300 to
    1,000 (each request holds a prefix of the same sequence, so its row is a row of the plain run):
    the three ranges of rows that take different product kernels."""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    folder, config = folder_for("xl4", dtype)
    V, n = config["vocab_size"], 1024
    tokens = helpers.random_tokens(n, V, seed=12)
    weights = _plain_weights(folder, config, dtype)
    hidden = plain.final_hidden(weights, config, tokens)  # [1024, 1600] float64
    wte = weights["model.wte.weight"].double()
    g = torch.Generator().manual_seed(3)
    cols = torch.randperm(V, generator=g)[:768].sort().values
    places = sorted({0, 1, 15, 16, 17, 127, 128, 129, 255, 256, 511, 512, 513, 991, 992, 1022, 1023}
                    | set(torch.randperm(n, generator=g)[:56].tolist()))
    assert len(places) >= 64
    want_cols = hidden @ wte[cols].t()            # every position, some columns
    want_rows = plain.tied_head(hidden[places], wte)  # some positions, every column
    scale = want_rows.abs().max().item()
    tol = TOL[dtype] * scale

    def check(got, positions, what):
        """``got``: logits [len(positions), V] of the engine at these positions of the sequence."""
        positions = list(positions)
        err = _err(got[:, cols], want_cols[positions])
        assert err <= tol, f"{what}: {err:.3g} against {tol:.3g} at some of positions {positions[0]} to {positions[-1]}"
        held = [(i, places.index(p)) for i, p in enumerate(positions) if p in places]
        if held:
            err = _err(got[[i for i, _ in held]], want_rows[[j for _, j in held]])
            assert err <= tol, f"{what}, whole vocabulary: {err:.3g} against {tol:.3g}"

    model, _ = load_model(folder, dtype=dtype)
    eng = Engine(model, dtype=dtype, page_size=16, n_pages=n // 16 + 4, max_requests=4)
    check(_run(eng, "whole", tokens, [n]), range(n), "whole")
    decoded = _run(eng, "decoded", tokens, [n - 32] + [1] * 32)
    check(decoded[n - 32:], range(n - 32, n), "last 32 one by one")
    check(decoded[: n - 32], range(n - 32), "all but the last 32 in one step")
    check(_run(eng, "portions", tokens, helpers.cuts_changing(n)), range(n), "portions of changing size")
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages
    del eng

    # one decode step of many requests at different contexts
    for n_req in (64, 40, 12):
        contexts = [300 + (700 * i) // (n_req - 1) for i in range(n_req)]  # 300 ... 1,000
        contexts = [c + (i % 5) for i, c in enumerate(contexts)]           # not all at a page's edge
        eng = Engine(model, dtype=dtype, page_size=16, n_pages=sum((c + 16) // 16 for c in contexts) + 2,
                     max_requests=n_req)
        for i, c in enumerate(contexts):
            eng.add_request(i)
        for first in range(0, n_req, 4):  # prompts four at a time, nothing wanted
            eng.step([StepEntry(i, tokens[: contexts[i]], []) for i in range(first, min(first + 4, n_req))])
        eng.cache.poison_free_pages()
        logits = eng.step([StepEntry(i, [tokens[c]], [0]) for i, c in enumerate(contexts)]).cpu()
        check(logits, contexts, f"a decode step of {n_req} requests")
        # (check() looks positions up one by one, so their order need not rise)
        eng.cache.check()
        del eng


def _replay(folder, dtype, out, steps, max_tokens):
    text = "".join(json.dumps(s) + "\n" for s in steps)
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
         "--out", str(out), "--max-tokens", str(max_tokens)],
        input=text, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.split("\n") if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    rows = [np.fromfile(os.path.join(out, f"{s['step']}.f32"), dtype="<f4").reshape(-1, 50257) for s in steps]
    return torch.from_numpy(np.concatenate(rows))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpt2_large_sizes_replayed_in_portions_of_1_7_64_and_1024(folder_for, tmp_path, dtype):
    """Width 1280, 20 heads, inner 5120, all 36 layers: a sequence of 1,024 tokens through
    ``bin/trace_run`` whole and in portions of 64, 7 and 1, logits at every position; all four
    runs in one call of the program, one request after the other, in a pool of 1,024 tokens."""
    folder, config = folder_for("large")
    n = 1024
    tokens = helpers.random_tokens(n, config["vocab_size"], seed=5)
    steps = []
    for chunk in (1024, 64, 7, 1):
        for i in range(0, n, chunk):
            c = min(chunk, n - i)
            steps.append({"step": len(steps), "entries": [{"id": f"c{chunk}", "tokens": tokens[i : i + c],
                                                           "want": list(range(c))}],
                          "end": [f"c{chunk}"] if i + c == n else []})
    rows = _replay(folder, dtype, tmp_path, steps, n)
    whole = rows[:n]
    scale = whole.abs().max().item()
    for k, chunk in enumerate((64, 7, 1), 1):
        assert _err(rows[k * n : (k + 1) * n], whole) <= TOL[dtype] * scale, f"portions of {chunk}"
    want = plain.forward(_plain_weights(folder, config, dtype), config, tokens[:96])
    assert _err(whole[:96], want) <= TOL[dtype] * want.abs().max().item(), "whole against the plain implementation"


def _mix64(x):
    m = (1 << 64) - 1
    x &= m
    x ^= x >> 30
    x = x * 0xBF58476D1CE4E5B9 & m
    x ^= x >> 27
    x = x * 0x94D049BB133111EB & m
    return x ^ (x >> 31)


def _fmix32(x):
    m = 0xFFFFFFFF
    x &= m
    x ^= x >> 16
    x = x * 0x85EBCA6B & m
    x ^= x >> 13
    x = x * 0xC2B2AE35 & m
    return x ^ (x >> 16)


def _gumbel(seed, counter, token):
    """The noise that the sampling kernel adds to token ``token``'s score in draw ``counter`` of a
    request with this seed (``csrc/sampling.hip``: a key from seed and counter, a uniform of 24
    bits hashed from key and token, ``-log(-log u)``)."""
    import math

    key = _mix64((seed & 0x7FFFFFFFFFFFFFFF) + 0x9E3779B97F4A7C15 * (counter + 1))
    x = _fmix32(((token + 1) * 0x9E3779B1 & 0xFFFFFFFF) ^ (key & 0xFFFFFFFF))
    x = _fmix32(x + (key >> 32))
    u = ((x >> 8) + 0.5) / 16777216.0
    return -math.log(-math.log(u))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gpt2_small_sizes_256_requests_under_load(folder_for, dtype):
    """Width 768, 12 heads, all 12 layers: 256 requests, prompts of 1 to 1,023 tokens, 1 to 255
    new tokens, temperature 0.8 with a seed per request, pages of 16 tokens, a pool of 24
    contexts for up to 48 running requests (so requests are pre-empted).  Every request
    finishes with ``min(max_new, positions - prompt)`` tokens; fourteen of them, run alone with
    room to spare, give the same tokens: all of them in float32.  In bfloat16 the logits of a
    row differ by rounding with the batch around it, and a draw that falls on the edge between
    two tokens may go the other way (from there on the two runs are different requests).  Such
    a first difference has to *be* on an edge: with the log-probabilities of the run alone and
    the draw's noise (which depends on seed, index and token only), the token that won alone
    and the token that won in the crowd have scores within twice the bfloat16 tolerance of the
    logits over the temperature.  Any number of requests may differ so; none otherwise."""
    from mlx_lm_amd.engine import StepEntry
    from mlx_lm_amd.generate import BatchGenerator, engine_for
    from mlx_lm_amd.sample_utils import make_sampler
    from mlx_lm_amd.utils import load_model

    folder, config = folder_for("small")
    P, V, n_req = config["n_positions"], config["vocab_size"], 256
    model, _ = load_model(folder, dtype=dtype)
    rng = random.Random(0)
    prompts = [[rng.randrange(V) for _ in range(rng.randrange(1, P))] for _ in range(n_req)]
    max_new = [rng.randrange(1, 256) for _ in range(n_req)]
    temp = 0.8
    sampler = make_sampler(temp=temp)

    def run(idx, cache_tokens, batch, keep_logprobs=False):
        eng = engine_for(model, max_requests=64, max_cache_tokens=cache_tokens)
        gen = BatchGenerator(model, sampler=sampler, completion_batch_size=batch, prefill_batch_size=4,
                             prefill_step_size=512, want_logprobs=keep_logprobs, engine=eng)
        uids = gen.insert([prompts[i] for i in idx], [max_new[i] for i in idx], seeds=[1000 + i for i in idx])
        out, reasons, lps = {u: [] for u in uids}, {}, {u: [] for u in uids}
        while responses := gen.next_generated():
            for r in responses:
                out[r.uid].append(r.token)
                if keep_logprobs:
                    lps[r.uid].append(r.logprobs)
                if r.finish_reason:
                    reasons[r.uid] = r.finish_reason
        eng.cache.check()
        assert eng.cache.free_pages() == eng.cache.n_pages
        return [out[u] for u in uids], [reasons.get(u) for u in uids], gen.scheduler.stats, [lps[u] for u in uids]

    idx = list(range(n_req))
    crowd, reasons, stats, _ = run(idx, 24 * P, 48)
    assert stats.preemptions > 0
    for i in idx:
        assert len(crowd[i]) == min(max_new[i], P - len(prompts[i])) and reasons[i] == "length", i
    # the size of the logits, for the tolerance of a score: one prompt through the engine
    eng = engine_for(model, max_requests=64, max_cache_tokens=2 * P)
    eng.add_request("scale")
    scale = eng.step([StepEntry("scale", prompts[0], [len(prompts[0]) - 1])]).abs().max().item()
    eng.end_request("scale")
    sample = idx[::19]
    assert len(sample) >= 12
    edges = 0
    for i in sample:
        alone, _, _, lps = run([i], 2 * P, 1, keep_logprobs=True)
        alone, lps = alone[0], lps[0]
        assert len(alone) == len(crowd[i])
        first = next((k for k, (x, y) in enumerate(zip(alone, crowd[i])) if x != y), None)
        if first is None:
            continue
        assert dtype == "bfloat16", f"request {i}: float32 differs at token {first}"
        x, y = alone[first], crowd[i][first]
        lp = lps[first].double().cpu()
        sx = lp[x].item() / temp + _gumbel(1000 + i, first, x)
        sy = lp[y].item() / temp + _gumbel(1000 + i, first, y)
        margin = 2 * TOL[dtype] * scale / temp
        print(f"{dtype}: request {i} differs from token {first} of {len(alone)} on: scores {sx:.4f} and {sy:.4f}, "
              f"allowed margin {margin:.4f}")
        # (x won alone: its score is the higher one there, up to the kernel's 32-bit arithmetic)
        assert -1e-3 <= sx - sy <= margin, f"request {i}, token {first}: {x} won alone by {sx - sy:.4f} over {y}"
        edges += 1
    print(f"{dtype}: {edges} of {len(sample)} requests met an edge")
