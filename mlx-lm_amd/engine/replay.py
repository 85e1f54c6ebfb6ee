"""Trace replay: feed given token ids through the model step by step, write logits.

Nothing is sampled.  The program drives the same model, step function, cache
manager and kernels that generation uses.

    trace_run --model DIR --dtype bfloat16|float32 --out DIR --max-tokens N

Steps come on standard input, one JSON object a line:

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step in which something is wanted, ``OUT/<step>.f32`` holds the logits
at the wanted places, in the order of the entries and of ``want``, as
little-endian float32 ``[wanted, vocab]``.  After every step a line
``done <step>`` is printed and flushed.

``want`` may also be ``"last"``, ``"all"`` or ``"none"``.  Instead of a folder,
``--config FILE --seed N`` names a configuration whose random weights are
written to a temporary folder first.  ``OUT/pages.jsonl`` gets a line per step
with the cache's state after it: pages free and held in every group, the most
held so far, live requests; ``--page-stats`` prints the same line, with
``pages `` before it, ahead of the step's ``done``.
"""

import argparse
import json
import os
import sys
import tempfile


def wanted_places(want, n_tokens):
    """``want`` as a list of places among a request's ``n_tokens`` tokens of the step."""
    if isinstance(want, str):
        if want == "all":
            return list(range(n_tokens))
        if want == "last":
            return [n_tokens - 1]
        if want == "none":
            return []
        raise SystemExit(f'"want" is a list of places or one of "last", "all", "none", not {want!r}')
    return list(want or [])


def page_statistics(engine, step):
    cm = engine.cache
    groups = [{"window": g.need.window, "free": g.pool.n_free, "held": g.pool.n_held,
               "high_water": g.pool.high_water} for g in cm.groups]
    return {"step": step, "page_size": cm.page_size, "n_pages": cm.n_pages, "groups": groups,
            "live_requests": len(cm.requests), "tokens_held": sum(rc.length for rc in cm.requests.values())}


def build_parser():
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", help="folder with config.json and model.safetensors")
    p.add_argument("--config", help="a config.json to draw random weights for (instead of --model)")
    p.add_argument("--seed", type=int, default=0, help="seed of the random weights (with --config)")
    p.add_argument("--scheme", choices=["a", "b"], default="b",
                   help="random weights: a = biases 0 and norms 1; b = all drawn (with --config)")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--out", required=True, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens that live requests hold at any time (each rounded up to 64)")
    p.add_argument("--page-size", "--block-size", dest="page_size", type=int, default=16,
                   help="tokens per cache page (16, 32 or 64)")
    p.add_argument("--num-pages", type=int, default=None,
                   help="pages of the pool (default: what --max-tokens needs)")
    p.add_argument("--page-stats", action="store_true", help="print every step's page statistics")
    p.add_argument("--max-requests", type=int, default=8, help="most requests live at a time")
    return p


def main(argv=None, stdin=None, stdout=None):
    args = build_parser().parse_args(argv)
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout
    if 64 % args.page_size:
        raise SystemExit("--page-size must divide 64")
    if (args.model is None) == (args.config is None):
        raise SystemExit("give --model DIR or --config FILE (with --seed)")
    os.makedirs(args.out, exist_ok=True)

    from ..utils import load_model
    from .step import Engine, StepEntry

    with tempfile.TemporaryDirectory() as tmp:
        folder = args.model
        if folder is None:
            from ..weights import write_model_folder

            with open(args.config) as fh:
                config = json.load(fh)
            write_model_folder(tmp, config, args.seed, args.scheme, dtype="float32")
            folder = tmp
        model, _ = load_model(folder, dtype=args.dtype)
    n_pages = args.num_pages or (args.max_tokens + 63) // 64 * (64 // args.page_size)
    engine = Engine(model, dtype=args.dtype, page_size=args.page_size, n_pages=n_pages,
                    max_requests=args.max_requests)

    stats_file = open(os.path.join(args.out, "pages.jsonl"), "w")
    for line in stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            if not e.get("tokens"):
                if e.get("want") not in (None, [], "none"):
                    raise SystemExit(f"step {step}: request {e['id']!r} wants logits but brings no tokens")
                continue  # a request that sits this step out
            if not engine.has_request(e["id"]):
                engine.add_request(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], wanted_places(e.get("want"), len(e["tokens"]))))
        logits = engine.step(entries)
        if logits is not None:
            data = logits.detach().to("cpu").contiguous().numpy().astype("<f4", copy=False)
            with open(os.path.join(args.out, f"{step}.f32"), "wb") as fh:
                fh.write(data.tobytes())
        for rid in rec.get("end", []):
            if engine.has_request(rid):
                engine.end_request(rid)
        stats = json.dumps(page_statistics(engine, step))
        stats_file.write(stats + "\n")
        stats_file.flush()
        if args.page_stats:
            stdout.write(f"pages {stats}\n")
        stdout.write(f"done {step}\n")
        stdout.flush()
    stats_file.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
