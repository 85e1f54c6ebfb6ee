"""The engine against the plain implementation: whole, decoded, in portions, mixed."""

import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import helpers
import plain_gpt2 as plain

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# max |engine - plain| as a fraction of max |plain logits|.  float32: the
# engine sums in float32 where the plain implementation has float64.
# bfloat16: activations are rounded to 8 bits of mantissa between the layers'
# matrix products (the plain side gets the same bfloat16-rounded matrices).
TOL = {"float32": 2e-5, "bfloat16": 2.5e-2}


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name in ("A", "B", "C"):
        for sharp in (0.0, 8.0):
            d = tmp_path_factory.mktemp(f"tiny{name}{int(sharp)}")
            out[(name, sharp)] = (str(d),) + helpers.make_folder(str(d), name, sharp)
    return out


def _engine(folder, dtype, n_pages, page_size=16, max_requests=8):
    from mlx_lm_amd.engine import Engine
    from mlx_lm_amd.utils import load_model

    model, _ = load_model(folder, dtype=dtype)
    return Engine(model, dtype=dtype, page_size=page_size, n_pages=n_pages, max_requests=max_requests)


def _plain_logits(weights, config, tokens, dtype):
    w = helpers.round_matrices_to_bf16(weights) if dtype == "bfloat16" else weights
    return plain.forward(w, config, tokens)


def _close(got, want, dtype, what=""):
    scale = want.abs().max().item()
    err = (got.double().cpu() - want).abs().max().item()
    assert err <= TOL[dtype] * scale, f"{what}: max error {err:.3e} against scale {scale:.3e}"


def _run(engine, rid, tokens, cuts, want_all=True):
    """Feed ``tokens`` in portions of the given sizes; logits at every position."""
    from mlx_lm_amd.engine import StepEntry

    engine.add_request(rid)
    rows, i = [], 0
    for n in cuts:
        part = tokens[i : i + n]
        rows.append(engine.step([StepEntry(rid, part, list(range(len(part))))]).clone())
        i += n
    assert i == len(tokens)
    engine.end_request(rid)
    return torch.cat(rows)


CASES = [("A", 0.0, 100), ("B", 0.0, 200), ("B", 8.0, 250), ("C", 8.0, 300), ("A", 8.0, 128)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,sharp,n", CASES)
def test_whole_decoded_and_portions(folders, dtype, name, sharp, n):
    folder, config, weights = folders[(name, sharp)]
    tokens = helpers.random_tokens(n, config["vocab_size"], seed=n)
    want = _plain_logits(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=(n + 15) // 16 + 2)
    whole = _run(eng, "whole", tokens, [n])
    _close(whole, want, dtype, "whole")
    decoded = _run(eng, "decoded", tokens, [n - 32] + [1] * 32)
    _close(decoded, want, dtype, "last 32 one by one")
    portions = _run(eng, "portions", tokens, helpers.cuts_changing(n))
    _close(portions, want, dtype, "portions of changing size")
    eng.cache.check()
    assert eng.cache.free_pages() == eng.cache.n_pages


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_first_tokens_and_long_decode(folders, dtype):
    """The first tokens of a sequence one by one, then decoding to the last position."""
    folder, config, weights = folders[("B", 8.0)]
    n = config["n_positions"]
    tokens = helpers.random_tokens(n, config["vocab_size"], seed=77)
    want = _plain_logits(weights, config, tokens, dtype)
    eng = _engine(folder, dtype, n_pages=n // 16)
    got = _run(eng, "r", tokens, [1] * n)
    _close(got[:8], want[:8], dtype, "first tokens")
    _close(got, want, dtype, "decoding every token")
    # one more token does not fit the model's positions
    from mlx_lm_amd.engine import StepEntry

    eng.add_request("full")
    eng.step([StepEntry("full", tokens, [])])
    with pytest.raises(ValueError, match="positions"):
        eng.step([StepEntry("full", [1], [0])])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("use_graphs", [False, True])
def test_thousands_of_keys_split_over_blocks(tmp_path, monkeypatch, dtype, use_graphs):
    """A prompt of 3,300 tokens in two portions, then 40 decoded tokens whose keys several blocks share,
    beside a request of a few dozen tokens."""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.ops import kernels
    from mlx_lm_amd.utils import load_model

    config, weights = helpers.make_folder(str(tmp_path), "LONG", 8.0)
    n, n_prompt = 3340, 3300
    tokens = helpers.random_tokens(n, config["vocab_size"], seed=31)
    want = _plain_logits(weights, config, tokens, dtype)
    model, _ = load_model(str(tmp_path), dtype=dtype)
    eng = Engine(model, dtype=dtype, page_size=16, n_pages=(n + 63) // 64 * 4 + 5, max_requests=2, use_graphs=use_graphs)
    eng.add_request("r")
    first = eng.step([StepEntry("r", tokens[:2000], [1999])])
    _close(first, want[1999:2000], dtype, "the first portion's last row")
    rows = [eng.step([StepEntry("r", tokens[2000:n_prompt], [n_prompt - 2001])]).clone()]
    # a short request decodes beside the long one: in one launch its rows take one part and the long one's several
    short = helpers.random_tokens(70, config["vocab_size"], seed=32)
    want_short = _plain_logits(weights, config, short, dtype)
    eng.add_request("s")
    short_rows = [eng.step([StepEntry("s", short[:30], [29])]).clone()]
    for i in range(n_prompt, n):
        both = eng.step([StepEntry("r", tokens[i : i + 1], [0]), StepEntry("s", short[i - n_prompt + 30 : i - n_prompt + 31], [0])])
        rows.append(both[:1].clone()), short_rows.append(both[1:].clone())
    assert eng.stats.key_splits_most > 1, "no step split a row's keys"
    _close(torch.cat(rows), want[n_prompt - 1 :], dtype, "decoded after 3,300 tokens")
    _close(torch.cat(short_rows), want_short[29:], dtype, "the short request beside it")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_decode_steps_by_class_of_length(tmp_path, dtype):
    """Decoding across the length from which a row's keys may be split: the recorded step of the
    shorter lengths is planned without splits, the next one with, and the logits do not notice."""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.ops import kernels
    from mlx_lm_amd.utils import load_model

    config, weights = helpers.make_folder(str(tmp_path), "LONG", 8.0)
    edge = kernels.rows_split_from()
    n_prompt, n = edge - 8, edge + 8
    tokens = helpers.random_tokens(n, config["vocab_size"], seed=33)
    want = _plain_logits(weights, config, tokens, dtype)
    model, _ = load_model(str(tmp_path), dtype=dtype)
    eng = Engine(model, dtype=dtype, page_size=16, n_pages=(n + 15) // 16 + 1, max_requests=2, use_graphs=True)
    eng.add_request("r")
    rows = [eng.step([StepEntry("r", tokens[:n_prompt], [n_prompt - 1])]).clone()]
    for i in range(n_prompt, n):
        rows.append(eng.step([StepEntry("r", tokens[i : i + 1], [0])]).clone())
    graphs = helpers.decode_graphs(eng, 1)
    assert len(graphs) == 2 and all(g.graph is not None for g in graphs)
    assert sorted(g.store.plan_positions for g in graphs) == [edge - 1, 2 * edge - 1]
    _close(torch.cat(rows), want[n_prompt - 1 :], dtype, "decoded across the edge of a class of length")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name,sharp", [("A", 8.0), ("B", 8.0), ("C", 0.0), ("C", 8.0)])
def test_mixed_batches_with_few_pages(folders, dtype, name, sharp):
    from mlx_lm_amd.engine import StepEntry

    folder, config, weights = folders[(name, sharp)]
    P = config["n_positions"]
    lengths = [min(P, n) for n in (100, 37, 128, 64, 90, 17, 120, 75)]
    tokens, steps = helpers.mixed_trace(config, seed=3, lengths=lengths)
    max_tokens = helpers.held(lengths, 4)
    eng = _engine(folder, dtype, n_pages=max_tokens // 16)
    got = {rid: [] for rid in tokens}
    used_pages = set()
    for s in steps:
        for e in s["entries"]:
            if not eng.has_request(e["id"]):
                eng.add_request(e["id"])
        eng.cache.poison_free_pages()
        logits = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        i = 0
        for e in s["entries"]:
            got[e["id"]].append(logits[i : i + len(e["want"])].clone())
            i += len(e["want"])
            used_pages.update(eng.cache.block_table(e["id"], 0))
        for rid in s["end"]:
            eng.end_request(rid)
        eng.cache.check()
    assert any(len(s["entries"]) >= 3 for s in steps)
    assert sum((n + 15) // 16 for n in lengths) > eng.cache.n_pages  # pages were used again
    for rid, toks in tokens.items():
        want = _plain_logits(weights, config, toks, dtype)
        _close(torch.cat(got[rid]), want, dtype, f"mixed, request {rid}")


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("name,sharp", [("B", 8.0), ("C", 0.0)])
@pytest.mark.parametrize("use_graphs", [False, True])
def test_split_sums_in_the_engine(folders, monkeypatch, name, sharp, use_graphs, dtype):
    """Projections that split K (forced here: tiny layers would not) leave their sums into the
    residual stream pending between the parts; the next norm adds them.  Mixed batches and
    recorded decode steps, against the plain implementation.  (In float32 only the kernel for up to
    64 rows splits K.)"""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.ops import kernels
    from mlx_lm_amd.utils import load_model

    monkeypatch.setattr(kernels, "force_splits", 2)
    folder, config, weights = folders[(name, sharp)]
    P = config["n_positions"]
    lengths = [min(P, n) for n in (100, 37, 128, 64, 90, 17)]
    tokens, steps = helpers.mixed_trace(config, seed=5, lengths=lengths)
    model, _ = load_model(folder, dtype=dtype)
    eng = Engine(model, dtype=dtype, page_size=16, n_pages=helpers.held(lengths, 4) // 16, max_requests=8,
                 use_graphs=use_graphs)
    got = {rid: [] for rid in tokens}
    for s in steps:
        for e in s["entries"]:
            if not eng.has_request(e["id"]):
                eng.add_request(e["id"])
        logits = eng.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        i = 0
        for e in s["entries"]:
            got[e["id"]].append(logits[i : i + len(e["want"])].clone())
            i += len(e["want"])
        for rid in s["end"]:
            eng.end_request(rid)
    assert eng.stats.settle_normed > 2 * len(model.layers)  # the fused kernel ran, in many steps
    # a few tokens of which only the last is wanted: the last block's sum is added without a norm,
    # since the final norm gathers its rows
    extra = helpers.random_tokens(11, config["vocab_size"], seed=77)
    eng.add_request("extra")
    before = eng.stats.settle_plain
    got["extra"] = [eng.step([StepEntry("extra", extra, [10])]).clone()]
    assert eng.stats.settle_plain == before + 1
    want = _plain_logits(weights, config, extra, dtype)[10:]
    _close(got.pop("extra")[0], want, dtype, "split sums, gathered rows")
    for rid, toks in tokens.items():
        want = _plain_logits(weights, config, toks, dtype)
        _close(torch.cat(got[rid]), want, dtype, f"split sums, request {rid}")


@pytest.mark.parametrize("page_size", [16, 32, 64])
def test_page_sizes_agree(folders, page_size):
    folder, config, weights = folders[("B", 8.0)]
    tokens = helpers.random_tokens(150, config["vocab_size"], seed=9)
    want = _plain_logits(weights, config, tokens, "float32")
    eng = _engine(folder, "float32", n_pages=4 * 64 // page_size, page_size=page_size)
    got = _run(eng, "r", tokens, [70, 2, 1, 1, 50, 26])
    _close(got, want, "float32", f"page size {page_size}")


def test_out_of_pages_is_an_error_and_takes_nothing(folders):
    from mlx_lm_amd.cache import OutOfPages
    from mlx_lm_amd.engine import StepEntry

    folder, config, _ = folders[("A", 0.0)]
    eng = _engine(folder, "float32", n_pages=4)
    eng.add_request("a")
    eng.add_request("b")
    eng.step([StepEntry("a", list(range(40)), [])])  # 3 pages
    with pytest.raises(OutOfPages):
        eng.step([StepEntry("a", [1], [0]), StepEntry("b", list(range(20)), [19])])
    eng.cache.check()
    assert eng.cache.free_pages() == 1
    assert eng.context_len("a") == 40 and eng.context_len("b") == 0
    out = eng.step([StepEntry("a", [1], [0]), StepEntry("b", list(range(10)), [9])])
    assert out.shape == (2, config["vocab_size"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(folders, tmp_path, dtype):
    """bin/trace_run as a user calls it: whole, decoded, in portions of changing size and mixed,
    from files; the three spellings of ``want``; the page statistics it leaves."""
    import json

    folder, config, weights = folders[("B", 8.0)]
    lengths = [90, 40, 130, 64, 70]
    tokens, steps = helpers.mixed_trace(config, seed=11, lengths=lengths, n_live=3)
    # a request whole, the same one with its last 32 tokens one by one, and in portions of changing size
    whole = helpers.random_tokens(120, config["vocab_size"], seed=5)

    def add(rid, toks, want, end=False):
        steps.append({"step": len(steps), "entries": [{"id": rid, "tokens": toks, "want": want}],
                      "end": [rid] if end else []})

    add("w", whole, "all", end=True)
    add("d", whole[:88], list(range(88)))
    for i in range(32):
        add("d", [whole[88 + i]], [0], end=i == 31)
    at = 0
    for n in helpers.cuts_changing(120):
        add("p", whole[at : at + n], "all", end=at + n == 120)
        at += n
    add("l", whole[:50], "none")
    add("l", whole[50:], "last", end=True)
    trace = tmp_path / "trace.jsonl"
    helpers.write_trace(trace, steps)
    out = tmp_path / "out"
    max_tokens = helpers.held(lengths + [128], 3)
    with open(trace) as fh:
        proc = subprocess.run(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
             "--out", str(out), "--max-tokens", str(max_tokens), "--page-stats"],
            stdin=fh, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = proc.stdout.split("\n")
    assert [l for l in lines if l.startswith("done")] == [f"done {s['step']}" for s in steps]
    V = config["vocab_size"]
    got = {}
    for s in steps:
        f = out / f"{s['step']}.f32"
        wants = [e["want"] for e in s["entries"]]
        if wants == ["none"]:
            assert not f.exists()
            continue
        data = np.fromfile(f, dtype="<f4").reshape(-1, V)
        i = 0
        for e in s["entries"]:
            n = {"all": len(e["tokens"]), "last": 1}.get(e["want"], len(e["want"])) if isinstance(e["want"], str) else len(e["want"])
            got.setdefault(e["id"], []).append(torch.from_numpy(data[i : i + n].copy()))
            i += n
        assert i == data.shape[0]
    last = got.pop("l")
    for rid in ("w", "d", "p"):
        tokens[rid] = whole
    for rid, toks in tokens.items():
        want = _plain_logits(weights, config, toks, dtype)
        _close(torch.cat(got[rid]), want, dtype, f"trace_run, request {rid}")
    _close(last[0], _plain_logits(weights, config, whole, dtype)[119:], dtype, 'want "last"')
    # page statistics: a line a step, in the file and (asked for) on standard output; nothing is
    # held at the end, and never more than the pool has
    stats = [json.loads(l) for l in open(out / "pages.jsonl")]
    assert [st["step"] for st in stats] == [s["step"] for s in steps]
    assert [json.loads(l[len("pages "):]) for l in lines if l.startswith("pages ")] == stats
    n_pages = max_tokens // 16
    assert all(st["n_pages"] == n_pages and g["held"] + g["free"] == n_pages for st in stats for g in st["groups"])
    assert stats[-1]["groups"][0]["held"] == 0 and stats[-1]["live_requests"] == 0
    assert 0 < max(g["high_water"] for g in stats[-1]["groups"]) <= n_pages


def test_trace_run_draws_its_own_weights(folders, tmp_path):
    """``--config FILE --seed N``: the same logits as from the folder that the random-weights
    mode writes for that configuration and seed."""
    import json

    from mlx_lm_amd.weights import write_model_folder

    config = dict(helpers.TINY_A)
    folder = tmp_path / "model"
    write_model_folder(str(folder), dict(config), 7, "b")
    (tmp_path / "cfg.json").write_text(json.dumps(config))
    toks = helpers.random_tokens(40, config["vocab_size"], seed=1)
    trace = json.dumps({"step": 0, "entries": [{"id": "a", "tokens": toks, "want": "all"}], "end": ["a"]}) + "\n"
    outs = []
    for i, source in enumerate((["--model", str(folder)], ["--config", str(tmp_path / "cfg.json"), "--seed", "7"])):
        out = tmp_path / f"out{i}"
        proc = subprocess.run(
            [sys.executable, os.path.join(ROOT, "bin", "trace_run"), *source, "--dtype", "float32", "--out", str(out),
             "--max-tokens", "64"], input=trace, capture_output=True, text=True, timeout=300)
        assert proc.returncode == 0, proc.stderr[-2000:]
        outs.append(np.fromfile(out / "0.f32", dtype="<f4"))
    assert outs[0].shape == (40 * config["vocab_size"],) and np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_decode_steps_equal_eager_ones(folders, dtype):
    """Decode steps replayed from a graph, with the program's own eager work between the
    replays (portions of other prompts, requests ending, pages used again), against
    the same trace run eagerly and against the plain implementation."""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    folder, config, weights = folders[("B", 8.0)]
    V = config["vocab_size"]
    model, _ = load_model(folder, dtype=dtype)
    seqs = {r: helpers.random_tokens(n, V, seed=60 + i) for i, (r, n) in enumerate(
        [("a", 120), ("b", 75), ("c", 200), ("d", 64)])}
    results = {}
    for use_graphs in (True, False):
        eng = Engine(model, dtype=dtype, page_size=16, n_pages=30, max_requests=4, use_graphs=use_graphs)
        assert eng.use_graphs == use_graphs
        got = {r: [] for r in seqs}
        fed = dict.fromkeys(seqs, 0)
        for r in ("a", "b", "c"):
            eng.add_request(r)
            n = len(seqs[r]) // 2
            got[r].append(eng.step([StepEntry(r, seqs[r][:n], list(range(n)))]).clone())
            fed[r] = n
        live = ["a", "b", "c"]
        step = 0
        while live:
            step += 1
            out = eng.step([StepEntry(r, [seqs[r][fed[r]]], [0]) for r in live])  # recorded
            for i, r in enumerate(live):
                got[r].append(out[i : i + 1].clone())
                fed[r] += 1
            for r in list(live):
                if fed[r] == len(seqs[r]):
                    eng.end_request(r)
                    live.remove(r)
            if step == 20:  # eager work between replays: a new request's prompt, in two portions
                eng.add_request("d")
                got["d"].append(eng.step([StepEntry("d", seqs["d"][:40], list(range(40)))]).clone())
                got["d"].append(eng.step([StepEntry("d", seqs["d"][40:63], list(range(23)))]).clone())
                fed["d"] = 63
                live.append("d")
            eng.cache.check()
        if use_graphs:
            assert sorted({n for n, _ in eng._graphs}) == [1, 2, 3, 4] and all(g.graph is not None for g in eng._graphs.values())
        results[use_graphs] = {r: torch.cat(v) for r, v in got.items()}
    for r, toks in seqs.items():
        want = _plain_logits(weights, config, toks, dtype)
        _close(results[True][r], want, dtype, f"recorded, request {r}")
        assert torch.equal(results[True][r], results[False][r]), r


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_recorded_steps_of_repeating_shapes(folders, dtype):
    """Portions of one size, alone and beside a decoding request, come back with the same shape: from
    the third time on such a step is replayed from a graph.  With so few pages that the replays see
    pages used again; every logit against the plain implementation."""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    folder, config, weights = folders[("B", 8.0)]
    V = config["vocab_size"]
    model, _ = load_model(folder, dtype=dtype)
    seqs = {r: helpers.random_tokens(n, V, seed=80 + i) for i, (r, n) in enumerate(
        [("a", 230), ("b", 200), ("c", 160)])}
    def portion(r, at, n):
        return StepEntry(r, seqs[r][at : at + n], list(range(n)))

    results = {}
    for record in (True, False):
        eng = Engine(model, dtype=dtype, page_size=16, n_pages=30, max_requests=4, record_prompt_steps=record)
        got = {r: [] for r in seqs}
        eng.add_request("a")
        for at in range(0, 200, 40):  # five steps of shape (40,)
            got["a"].append(eng.step([portion("a", at, 40)]).clone())
        eng.add_request("b")
        for i in range(5):  # five of shape (1, 40)
            out = eng.step([portion("a", 200 + i, 1), portion("b", 40 * i, 40)])
            got["a"].append(out[:1].clone())
            got["b"].append(out[1:].clone())
        for i in range(5, 30):  # decode steps
            got["a"].append(eng.step([portion("a", 200 + i, 1)]).clone())
        eng.end_request("a")
        eng.end_request("b")
        eng.cache.poison_free_pages()
        eng.add_request("c")
        for at in range(0, 160, 40):  # shape (40,) again, replayed, on pages that a and b held
            got["c"].append(eng.step([portion("c", at, 40)]).clone())
        eng.cache.check()
        recorded = {k: g for k, g in eng._step_graphs.items() if g.graph is not None}
        assert set(recorded) == ({((40,), 40, True), ((1, 40), 41, True)} if record else set())
        results[record] = {r: torch.cat(v) for r, v in got.items()}
    for r, toks in seqs.items():
        n = results[True][r].shape[0]
        want = _plain_logits(weights, config, toks[:n], dtype)
        _close(results[True][r], want, dtype, f"recorded shapes, request {r}")
        assert torch.equal(results[True][r], results[False][r]), r  # the same launches, replayed


def test_a_dropped_engine_frees_its_graphs_at_once(folders):
    """An engine and its recorded graphs form no reference cycle: dropping the engine frees them
    there and then.  (Left to the cycle collector, a graph could be destroyed while another
    engine records one, which HIP refuses with an error that ends the process.)"""
    import gc
    import weakref

    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    folder, config, _ = folders[("A", 8.0)]
    model, _ = load_model(folder, dtype="bfloat16")
    gc.collect()
    gc.disable()
    try:
        eng = Engine(model, dtype="bfloat16", page_size=16, n_pages=8, max_requests=4, record_prompt_steps=True)
        eng.add_request("a")
        for at in range(0, 12, 3):  # the shape (3,) four times: recorded from the third on
            eng.step([StepEntry("a", [1 + at, 2 + at, 3 + at], [2])])
        for t in range(3):
            eng.step([StepEntry("a", [20 + t], [0])])
        refs = [weakref.ref(eng), weakref.ref(helpers.decode_graphs(eng, 1)[0])] + [weakref.ref(g) for g in eng._step_graphs.values()]
        assert len(refs) == 3 and helpers.decode_graphs(eng, 1)[0].graph is not None
        del eng
        assert all(r() is None for r in refs)
    finally:
        gc.enable()


@pytest.mark.parametrize("use_graphs", [True, False])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_tokens_fed_on_the_device(folders, dtype, use_graphs):
    """A decode step may take its tokens from the sampler's device array (the host reads them a
    step later): same logits, bit for bit, as with the tokens passed through the host.  Rows of the
    fed array in another order than the entries, a host token beside fed ones, and a portion of a
    prompt beside them (a step that is not replayed from a graph)."""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.sample_utils import Sampler
    from mlx_lm_amd.sampling import sample_batch
    from mlx_lm_amd.utils import load_model

    folder, config, weights = folders[("B", 8.0)]
    V = config["vocab_size"]
    model, _ = load_model(folder, dtype=dtype)
    prompts = {r: helpers.random_tokens(n, V, seed=90 + i) for i, (r, n) in enumerate([("a", 33), ("b", 70), ("c", 5)])}
    late = helpers.random_tokens(40, V, seed=99)
    greedy = [Sampler()] * 3

    def run(feed):
        eng = Engine(model, dtype=dtype, page_size=16, n_pages=40, max_requests=4, use_graphs=use_graphs)
        rows = []
        for r, toks in prompts.items():
            eng.add_request(r)
            rows.append(eng.step([StepEntry(r, toks, [len(toks) - 1])])[0].clone())
        logits = torch.stack(rows)
        history, kept = [], []
        for step in range(24):
            tokens, _ = sample_batch(logits, greedy, [0, 1, 2], [step] * 3)
            order = ["c", "a", "b"] if step % 2 else ["a", "b", "c"]  # entries in another order than the rows
            row_of = {"a": 0, "b": 1, "c": 2}
            if feed:
                entries = [StepEntry(r, [0], [0], fed_row=row_of[r]) for r in order]
                if step % 5 == 4:  # one token through the host beside fed ones
                    r = order[1]
                    entries[1] = StepEntry(r, [int(tokens[row_of[r]])], [0])
            else:
                host = tokens.tolist()
                entries = [StepEntry(r, [host[row_of[r]]], [0]) for r in order]
            if step == 10:  # a portion of a new prompt beside the decoding requests: an eager step
                eng.add_request("late")
                entries.append(StepEntry("late", late, []))
            out = eng.step(entries, fed=tokens if feed else None)
            history.append(tokens.clone())
            logits = torch.stack([out[order.index(r)] for r in ("a", "b", "c")]).clone()
            kept.append(logits)
        return torch.stack(history), torch.stack(kept)

    tokens_host, logits_host = run(False)
    tokens_fed, logits_fed = run(True)
    assert torch.equal(tokens_host, tokens_fed)
    assert torch.equal(logits_host, logits_fed)
    # and the tokens are what the plain model decodes greedily
    want = plain.greedy_generate(helpers.round_matrices_to_bf16(weights) if dtype == "bfloat16" else weights,
                                 config, prompts["c"], 6)
    assert tokens_host[:6, 2].tolist() == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("use_graphs", [True, False])
def test_trim_and_regenerate_across_a_page_edge(folders, dtype, use_graphs):
    """Decode, trim three tokens back over a page's edge, let another request take the page that
    went back, decode the same tokens again: same logits as before and as the plain implementation's
    (the reference's test of trimming, tests/test_prompt_cache.py:266-294, through this engine).
    Under recorded decode steps the request's row of the block table must be copied again: the
    table has its old length but another page, and the old page is the other request's now."""
    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model

    folder, config, weights = folders[("B", 8.0)]
    V = config["vocab_size"]
    model, _ = load_model(folder, dtype=dtype)
    eng = Engine(model, dtype=dtype, page_size=16, n_pages=8, max_requests=4, use_graphs=use_graphs)
    a = helpers.random_tokens(56, V, seed=301)
    b = helpers.random_tokens(40, V, seed=302)
    want_a, want_b = (_plain_logits(weights, config, t, dtype) for t in (a, b))

    eng.add_request("a")
    eng.step([StepEntry("a", a[:44], [])])
    first = [eng.step([StepEntry("a", [a[i]], [0])]).clone() for i in range(44, 50)]  # crosses 48
    _close(torch.cat(first), want_a[44:50], dtype, "before the trim")
    page_beyond_edge = eng.cache.requests["a"].blocks[0][3]
    assert eng.trim("a", 3) == 3 and eng.context_len("a") == 47
    assert len(eng.cache.requests["a"].blocks[0]) == 3
    # another request takes the page that went back (the pool hands out the last one returned)
    eng.add_request("b")
    got_b = [eng.step([StepEntry("b", b[:10], list(range(10)))]).clone()]
    assert eng.cache.requests["b"].blocks[0] == [page_beyond_edge]
    # the same tokens again, decoded one by one: position 48 needs a page, and gets another one
    again = [eng.step([StepEntry("a", [a[i]], [0])]).clone() for i in range(47, 56)]
    assert eng.cache.requests["a"].blocks[0][3] != page_beyond_edge
    _close(torch.cat(again), want_a[47:56], dtype, "after the trim")
    for x, y in zip(first[3:], again):  # positions 47, 48, 49 were computed before the trim too
        assert torch.equal(x, y)
    # and the other request's page was left alone
    got_b += [eng.step([StepEntry("b", [b[i]], [0])]).clone() for i in range(10, 40)]
    _close(torch.cat(got_b), want_b, dtype, "the request that took the page")
    if use_graphs:
        assert all(g.graph is not None for g in helpers.decode_graphs(eng, 1)) and helpers.decode_graphs(eng, 1)
    # trimming more than there is drops everything (tests/test_prompt_cache.py:259-264)
    assert eng.trim("a", 1000) == 56 and eng.context_len("a") == 0
    eng.end_request("a")
    eng.end_request("b")
    eng.cache.check()
    assert eng.cache.free_pages() == 8
