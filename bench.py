"""Decode and prefill throughput of GPT-2 XL layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--dtype bfloat16]

Prints one JSON line.  ``value`` is decoded tokens a second at the given batch
(default 8): K timed decode steps after W untimed ones, every request starting
from a 512-token prompt (the reference's benchmark draws uniform random
prompts and switches end-of-sequence off, mlx_lm/benchmark.py:118-124).
``prefill`` is one step of 2 x 1,024 prompt tokens (the best of five: a step
whose shape keeps coming back is replayed from its recorded graph, as in the
serving path); ``points`` holds decode at
batch 1 and 64; ``roofline`` the bytes a decode step has to read over its time.
Weights are random (seeded), data synthetic.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X, published: HBM3E 8 TB/s; dense MFMA bf16/fp16 2.5 PFLOP/s, fp32 157.3 TFLOP/s
PEAK_HBM_GBS = 8000.0
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}

XL = dict(model_type="gpt2", n_layer=48, n_embd=1600, n_head=25, n_inner=6400, vocab_size=50257,
          n_positions=1024, n_ctx=1024, layer_norm_epsilon=1e-5, activation_function="gelu_new")


def build_model(config, dtype, seed):
    """Random weights straight onto the GPU, through the architecture's own
    random_weights, sanitize and strict placement (no file in between)."""
    from mlx_lm_amd.config import get_model_classes
    from mlx_lm_amd.weights.loader import place_tensors, resolve_dtype

    model_cls, args_cls = get_model_classes(config)
    args = args_cls.from_dict(config)
    model = model_cls(args)
    tensors = model.sanitize(model_cls.random_weights(args, seed, "a"))
    model.decoder.load_tensors(place_tensors(model.decoder.expected_tensors(), tensors, dtype, "cuda:0"))
    model.dtype = resolve_dtype(dtype)
    model.device = "cuda:0"
    return model, args


def weight_bytes(model):
    """Bytes of every tensor a decode step uses once (the position table is read row-wise: left out)."""
    total = 0
    seen = {}
    for part in model.decoder.parts():
        for name, spec in part.tensors().items():
            seen[name] = spec
    import torch

    esize = torch.empty((), dtype=model.dtype).element_size()
    for name, spec in seen.items():
        if name.endswith("wpe.weight"):
            continue
        n = 1
        for s in spec.shape:
            n *= s
        total += n * (esize if spec.role == "matrix" else 4)
    return total


def prefill_flops(args, n_seqs, seq_len):
    D, F, L, V = args.n_embd, args.n_inner, args.n_layer, args.vocab_size
    per_token = 2 * L * (3 * D * D + D * D + 2 * D * F)
    attn = n_seqs * L * 4 * D * seq_len * (seq_len + 1) / 2  # causal: half of QK^T and PV
    head = 2 * n_seqs * D * V
    return per_token * n_seqs * seq_len + attn + head


def run_decode(engine, batch, prompt_len, steps, warmup, vocab, seed):
    """`batch` requests of `prompt_len` tokens through the scheduler (the loop that generation uses:
    a step is launched while the host reads the tokens of the one before); times `steps` decode steps."""
    import torch

    from mlx_lm_amd.engine.scheduler import Request, Scheduler
    from mlx_lm_amd.generate import make_sample_fn

    g = torch.Generator().manual_seed(seed)
    prompts = torch.randint(0, vocab, (batch, prompt_len), generator=g).tolist()
    # prompts go in four at a time to bound the step's scratch memory
    sched = Scheduler(engine, make_sample_fn(), max_num_seqs=batch,
                      max_num_batched_tokens=4 * prompt_len + batch, prefill_step_size=prompt_len)
    rids = [("bench", batch, i) for i in range(batch)]
    for i, rid in enumerate(rids):
        sched.add(Request(rid, prompts[i], max_tokens=10**6, seed=i))  # greedy; the timed steps end it
    while sched.waiting or not all(r.decoding for r in sched.running):
        sched.step()
    for _ in range(warmup):
        sched.step()
    torch.cuda.synchronize()
    ctx0 = sum(engine.context_len(rid) for rid in rids) / batch
    t0 = time.perf_counter()
    n_out = 0
    for _ in range(steps):
        n_out += len(sched.step())  # every step hands out one token per request
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ctx1 = sum(engine.context_len(rid) for rid in rids) / batch
    if n_out != batch * steps:
        raise RuntimeError(f"{n_out} tokens came out of {steps} steps of {batch} requests")
    for rid in rids:
        sched.abort(rid)
    return dt, (ctx0 + ctx1) / 2


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=128)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--layers", type=int, default=XL["n_layer"], help="run fewer layers than GPT-2 XL has")
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--no-points", action="store_true", help="skip batch 1 and 64")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU; this engine does not run on several (asked for %d)" % a.gpus)
        sys.exit(2)

    import torch

    from mlx_lm_amd.engine import Engine, StepEntry

    config = dict(XL)
    config["n_layer"] = a.layers
    t_build = time.perf_counter()
    model, args = build_model(config, a.dtype, seed=2)
    print(f"[bench] model built in {time.perf_counter() - t_build:.1f} s", file=sys.stderr, flush=True)
    P, V = args.n_positions, args.vocab_size
    steps = min(a.steps, P - a.prompt_len - a.warmup)
    # (as the serving path makes it, generate.engine_for: steps of a shape that keeps coming back are recorded)
    engine = Engine(model, dtype=a.dtype, page_size=16, max_tokens=64 * P, max_requests=64, record_prompt_steps=True)
    esize = 2 if a.dtype == "bfloat16" else 4
    kv_bytes_per_token = 2 * args.n_embd * args.n_layer * esize
    w_bytes = weight_bytes(model)

    # prefill: 2 x 1,024 tokens in one step
    g = torch.Generator().manual_seed(0)
    n_seqs, seq_len = 2, 1024
    prompts = torch.randint(0, V, (n_seqs, seq_len), generator=g).tolist()
    pre_ms = []
    for trial in range(5):  # the third records the step, the later ones replay it
        for i in range(n_seqs):
            engine.add_request(("pre", i))
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step([StepEntry(("pre", i), prompts[i], [seq_len - 1]) for i in range(n_seqs)])
        torch.cuda.synchronize()
        pre_ms.append((time.perf_counter() - t0) * 1e3)
        for i in range(n_seqs):
            engine.end_request(("pre", i))
    pre = min(pre_ms[1:])
    flops = prefill_flops(args, n_seqs, seq_len)
    prefill = {"value": round(n_seqs * seq_len / (pre / 1e3), 1), "tokens": n_seqs * seq_len,
               "ms": round(pre, 3), "frac": round(flops / (pre / 1e3) / PEAK_FLOPS[a.dtype], 4)}
    print(f"[bench] prefill {prefill} (trials, ms: {[round(t, 2) for t in pre_ms]})", file=sys.stderr, flush=True)

    results = {}
    batches = [a.batch] if a.no_points else sorted({1, a.batch, 64})
    for b in batches:
        k = steps if b == a.batch else min(steps, 64)
        dt, mean_ctx = run_decode(engine, b, a.prompt_len, k, a.warmup, V, seed=b)
        results[b] = (b * k / dt, dt / k * 1e3, mean_ctx, k)
        print(f"[bench] decode batch {b}: {results[b][0]:.1f} tok/s, {results[b][1]:.3f} ms/step",
              file=sys.stderr, flush=True)

    tps, ms, mean_ctx, k = results[a.batch]
    step_bytes = w_bytes + a.batch * mean_ctx * kv_bytes_per_token
    achieved = step_bytes / (ms / 1e3) / 1e9
    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens (GPT-2 XL)",
        "value": round(tps, 1), "unit": "tokens/s", "n_gpus": 1, "steps": k, "warmup": a.warmup,
        "ms_per_step": round(ms, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
        "data": "synthetic uniform random token ids, random weights (seed 2)",
        "config": {"model": "gpt2-xl layer sizes", "n_layer": a.layers, "n_layer_full": XL["n_layer"],
                   "n_embd": args.n_embd, "n_head": args.n_head, "n_inner": args.n_inner,
                   "vocab_size": V, "n_positions": P, "global_batch": a.batch,
                   "seq_len": P, "prompt_len": a.prompt_len, "page_size": 16, "parallelism": "none"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM_GBS, 4)},
        "points": {f"decode_b{b}": round(results[b][0], 1) for b in results if b in (1, 64)},
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
