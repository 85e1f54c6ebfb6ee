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
"""

import argparse
import json
import os
import sys


def build_parser():
    p = argparse.ArgumentParser(prog="trace_run", description=__doc__.split("\n\n")[0])
    p.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    p.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    p.add_argument("--out", required=True, help="folder for <step>.f32 files")
    p.add_argument("--max-tokens", type=int, required=True,
                   help="most tokens that live requests hold at any time (each rounded up to 64)")
    p.add_argument("--page-size", type=int, default=16, help="tokens per cache page (16, 32 or 64)")
    p.add_argument("--max-requests", type=int, default=8, help="most requests live at a time")
    return p


def main(argv=None, stdin=None, stdout=None):
    args = build_parser().parse_args(argv)
    stdin = stdin or sys.stdin
    stdout = stdout or sys.stdout
    if 64 % args.page_size:
        raise SystemExit("--page-size must divide 64")
    os.makedirs(args.out, exist_ok=True)

    from ..utils import load_model
    from .step import Engine, StepEntry

    model, _ = load_model(args.model, dtype=args.dtype)
    n_pages = (args.max_tokens + 63) // 64 * (64 // args.page_size)
    engine = Engine(model, dtype=args.dtype, page_size=args.page_size, n_pages=n_pages,
                    max_requests=args.max_requests)

    for line in stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            if not e.get("tokens"):
                if e.get("want"):
                    raise SystemExit(f"step {step}: request {e['id']!r} wants logits but brings no tokens")
                continue  # a request that sits this step out
            if not engine.has_request(e["id"]):
                engine.add_request(e["id"])
            entries.append(StepEntry(e["id"], e["tokens"], e.get("want", [])))
        logits = engine.step(entries)
        if logits is not None:
            data = logits.detach().to("cpu").contiguous().numpy().astype("<f4", copy=False)
            with open(os.path.join(args.out, f"{step}.f32"), "wb") as fh:
                fh.write(data.tobytes())
        for rid in rec.get("end", []):
            if engine.has_request(rid):
                engine.end_request(rid)
        stdout.write(f"done {step}\n")
        stdout.flush()
    return 0


if __name__ == "__main__":
    sys.exit(main())
