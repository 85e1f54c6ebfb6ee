"""Decode and prefill throughput of GPT-2 XL layer sizes on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--dtype bfloat16]

Prints one JSON line.  ``value`` is decoded tokens a second at the given batch (default 8):
K timed decode steps, every request starting from a 512-token prompt, so that the first timed
step runs at context 512 and, with the default K, the last at the model's last position but one (511 steps)
(the reference's benchmark draws uniform random prompts and switches end-of-sequence off,
mlx_lm/benchmark.py:118-124; it warms up, then times five trials and reports their mean,
mlx_lm/benchmark.py:152-176).  The W warm-up steps run before, on requests of their own, so
that they do not move the timed steps' context.  ``config`` gives the context range as
``ctx_from``/``ctx_to``.  ``prefill`` is one step of 2 x 1,024 prompt tokens: W untimed
warm-up trials, three at least (a step whose shape keeps coming back is replayed from its
recorded graph, as in the serving path: the third trial records it), then the mean of five
timed ones, each listed in ``trials_ms``.
``points`` holds decode at batch 1, 16, 32, 48 and 64 over the same steps and, for batch 1, 8 and
64, at context 1,000; ``roofline`` the bytes a decode step has to read (every weight once, the live
requests' keys and values at each step's context) over its time, ``roofline_points`` the same
fraction for every point.  Times are the host's clock around the steps with the GPU drained on
both sides; ``gpu_ms_per_step`` (and ``prefill.gpu_ms``) is the same stretch between two events
on the GPU's stream, the reference's way of timing apart (mlx_lm/benchmark.py:152-176 times with
the host's clock around an evaluated result).  Weights are random (seeded), data synthetic.

``--n-positions 8192`` is a mode of its own for long contexts: the same layer sizes with 8,192
positions and, unless ``--layers`` says otherwise, 12 of the 48 layers (``config`` names both);
``value`` is decode at batch 8 from context 7,000, ``points`` hold batch 1 and 8 at contexts 4,000
and 7,000, ``prefill`` is one prompt of 8,192 tokens.
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
    """Random weights under a checkpoint's names, loaded the way a folder's are."""
    from mlx_lm_amd.config import get_model_classes
    from mlx_lm_amd.utils import model_from_tensors

    model_cls, args_cls = get_model_classes(config)
    tensors = model_cls.random_weights(args_cls.from_dict(config), seed, "a")
    model = model_from_tensors(config, tensors, dtype=dtype, device="cuda:0")
    return model, model.args


def prefill_flops(args, n_seqs, seq_len):
    D, F, L, V = args.n_embd, args.n_inner, args.n_layer, args.vocab_size
    per_token = 2 * L * (3 * D * D + D * D + 2 * D * F)
    attn = n_seqs * L * 4 * D * seq_len * (seq_len + 1) / 2  # causal: half of QK^T and PV
    head = 2 * n_seqs * D * V
    return per_token * n_seqs * seq_len + attn + head


def _scheduler(engine, batch, prompt_len):
    from mlx_lm_amd.engine.scheduler import Scheduler
    from mlx_lm_amd.generate import make_sample_fn

    # all prompts go in one step, so that every request decodes from the same context on
    return Scheduler(engine, make_sample_fn(), max_num_seqs=batch,
                     max_num_batched_tokens=batch * (prompt_len + 1), prefill_step_size=prompt_len)


def _start(engine, sched, batch, prompt_len, vocab, seed, tag):
    import torch

    from mlx_lm_amd.engine.scheduler import Request

    g = torch.Generator().manual_seed(seed)
    prompts = torch.randint(0, vocab, (batch, prompt_len), generator=g).tolist()
    requests = [Request((tag, batch, i), prompts[i], max_tokens=10**6, seed=i)  # greedy; the caller ends it
                for i in range(batch)]
    for r in requests:
        sched.add(r)
    while sched.waiting or not all(r.decoding for r in sched.running):
        sched.step()
    return requests


def run_decode(engine, batch, prompt_len, steps, warmup, vocab, seed):
    """``batch`` requests of ``prompt_len`` tokens through the scheduler (the loop that generation
    uses: a step is launched while the host reads the tokens of the one before); times ``steps``
    decode steps.  Returns ``(seconds, contexts)``: the context each timed step ran at."""
    import torch

    sched = _scheduler(engine, batch, prompt_len)
    if warmup > 0:  # on requests of their own, so that the timed steps start at the prompt's end
        requests = _start(engine, sched, batch, prompt_len, vocab, seed + 1000, "warm")
        for _ in range(warmup):
            sched.step()
        torch.cuda.synchronize()
        for r in requests:
            sched.abort(r.request_id)
        while sched.has_work:
            sched.step()
    requests = _start(engine, sched, batch, prompt_len, vocab, seed, "bench")
    torch.cuda.synchronize()
    ctx0 = engine.context_len(requests[0].engine_id)
    first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    first.record()
    n_out = 0
    for _ in range(steps):
        n_out += len(sched.step())  # every step hands out one token per request
    last.record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    run_decode.gpu_seconds = first.elapsed_time(last) / 1e3
    if n_out != batch * steps:
        raise RuntimeError(f"{n_out} tokens came out of {steps} steps of {batch} requests")
    for r in requests:  # (a request that has reached the model's last position is over already)
        if r.live:
            sched.abort(r.request_id)
    while sched.has_work:
        sched.step()
    # steps overlap: the first timed call launches the step at the prompt's end, and every call
    # hands out the tokens of the step before, so `steps` calls ran `steps` steps
    return dt, list(range(ctx0, ctx0 + steps))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=512)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16")
    ap.add_argument("--layers", type=int, default=None, help="run fewer layers than GPT-2 XL has")
    ap.add_argument("--prompt-len", type=int, default=None)
    ap.add_argument("--n-positions", type=int, default=XL["n_positions"],
                    help="positions of the model; 8192: the long-context mode (12 layers unless --layers is given)")
    ap.add_argument("--no-points", action="store_true", help="skip the other batch sizes and contexts")
    a = ap.parse_args()
    long_mode = a.n_positions != XL["n_positions"]
    if a.layers is None:
        a.layers = 12 if long_mode else XL["n_layer"]
    if a.prompt_len is None:
        a.prompt_len = a.n_positions * 7000 // 8192 if long_mode else 512
    if a.gpus != 1:
        print("bench.py measures one GPU; this engine does not run on several (asked for %d)" % a.gpus)
        sys.exit(2)

    import torch

    from mlx_lm_amd.engine import Engine, StepEntry

    config = dict(XL)
    config["n_layer"] = a.layers
    config["n_positions"] = config["n_ctx"] = a.n_positions
    t_build = time.perf_counter()
    model, args = build_model(config, a.dtype, seed=2)
    print(f"[bench] model built in {time.perf_counter() - t_build:.1f} s", file=sys.stderr, flush=True)
    P, V = args.n_positions, args.vocab_size
    # the step after a prompt of p tokens runs at context p; the token that takes the last position
    # (P - 1) is never fed, so the last step runs at context P - 2
    steps = max(1, min(a.steps, P - 1 - a.prompt_len))
    # (as the serving path makes it, generate.engine_for: steps of a shape that keeps coming back are recorded)
    engine = Engine(model, dtype=a.dtype, page_size=16, max_tokens=(8 if long_mode else 64) * P, max_requests=64,
                    record_prompt_steps=True)
    esize = 2 if a.dtype == "bfloat16" else 4
    kv_bytes_per_token = engine.cache.bytes_per_token()
    w_bytes = model.decoder.bytes_read_per_step(esize)

    # prefill: 2 x 1,024 tokens in one step (the long-context mode: one prompt of all the positions)
    g = torch.Generator().manual_seed(0)
    n_seqs, seq_len = (1, P) if long_mode else (2, 1024)
    prompts = torch.randint(0, V, (n_seqs, seq_len), generator=g).tolist()
    pre_ms, pre_gpu_ms = [], []
    # (the third sighting of the shape records it; the warm-up trials after it and the timed ones replay)
    warm_trials, timed_trials = max(3, a.warmup), 5
    for trial in range(warm_trials + timed_trials):
        for i in range(n_seqs):
            engine.add_request(("pre", i))
        torch.cuda.synchronize()
        first, last = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        first.record()
        engine.step([StepEntry(("pre", i), prompts[i], [seq_len - 1]) for i in range(n_seqs)])
        last.record()
        torch.cuda.synchronize()
        pre_ms.append((time.perf_counter() - t0) * 1e3)
        pre_gpu_ms.append(first.elapsed_time(last))
        for i in range(n_seqs):
            engine.end_request(("pre", i))
    timed = pre_ms[warm_trials:]
    pre = sum(timed) / len(timed)
    flops = prefill_flops(args, n_seqs, seq_len)
    prefill = {"value": round(n_seqs * seq_len / (pre / 1e3), 1), "tokens": n_seqs * seq_len,
               "ms": round(pre, 3), "frac": round(flops / (pre / 1e3) / PEAK_FLOPS[a.dtype], 4),
               "trials_ms": [round(t, 3) for t in timed],
               "gpu_ms": round(sum(pre_gpu_ms[warm_trials:]) / timed_trials, 3)}
    print(f"[bench] prefill {prefill} (warm-up trials, ms: {[round(t, 2) for t in pre_ms[:warm_trials]]})",
          file=sys.stderr, flush=True)

    def measure(batch, prompt_len, k):
        dt, contexts = run_decode(engine, batch, prompt_len, k, a.warmup, V, seed=batch)
        ms = dt / k * 1e3
        gpu_ms = run_decode.gpu_seconds / k * 1e3
        step_bytes = w_bytes + batch * (sum(contexts) / len(contexts)) * kv_bytes_per_token
        gbs = step_bytes / (ms / 1e3) / 1e9
        print(f"[bench] decode batch {batch}, context {contexts[0]} to {contexts[-1]}: {batch * k / dt:.1f} tok/s, "
              f"{ms:.3f} ms/step ({gpu_ms:.3f} between events on the GPU), {gbs:.0f} GB/s", file=sys.stderr, flush=True)
        return {"tps": batch * k / dt, "ms": ms, "gpu_ms": gpu_ms, "gbs": gbs, "ctx": (contexts[0], contexts[-1]), "k": k}

    main_point = measure(a.batch, a.prompt_len, steps)
    points, fracs = {}, {f"decode_b{a.batch}": round(main_point["gbs"] / PEAK_HBM_GBS, 4)}
    if not a.no_points and long_mode:
        for b in sorted({1, a.batch}):
            for ctx in (P * 4000 // 8192, P * 7000 // 8192):
                r = main_point if (b, ctx) == (a.batch, a.prompt_len) else measure(b, ctx, min(steps, 128, P - 1 - ctx))
                points[f"decode_b{b}_ctx{ctx}"] = round(r["tps"], 1)
                fracs[f"decode_b{b}_ctx{ctx}"] = round(r["gbs"] / PEAK_HBM_GBS, 4)
    elif not a.no_points:
        for b in (1, 16, 32, 48, 64):
            r = main_point if b == a.batch else measure(b, a.prompt_len, steps)
            points[f"decode_b{b}"] = round(r["tps"], 1)
            fracs[f"decode_b{b}"] = round(r["gbs"] / PEAK_HBM_GBS, 4)
        late = min(1000, P - 8)
        for b in sorted({1, a.batch, 64}):
            r = measure(b, late, min(steps, P - 1 - late))
            points[f"decode_b{b}_ctx{late}"] = round(r["tps"], 1)
            fracs[f"decode_b{b}_ctx{late}"] = round(r["gbs"] / PEAK_HBM_GBS, 4)

    line = {
        "metric": "decode tok/s at batch 1/8/64; prefill tok/s at 2,048 tokens (GPT-2 XL)",
        "value": round(main_point["tps"], 1), "unit": "tokens/s", "n_gpus": 1, "steps": main_point["k"],
        "warmup": a.warmup, "ms_per_step": round(main_point["ms"], 4),
        "gpu_ms_per_step": round(main_point["gpu_ms"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if a.dtype == "bfloat16" else "fp32",
        "data": "synthetic uniform random token ids, random weights (seed 2)",
        "config": {"model": "gpt2-xl layer sizes", "n_layer": a.layers, "n_layer_full": XL["n_layer"],
                   "n_embd": args.n_embd, "n_head": args.n_head, "n_inner": args.n_inner,
                   "vocab_size": V, "n_positions": P, "layer_norm_epsilon": args.layer_norm_epsilon,
                   "global_batch": a.batch, "seq_len": P, "prompt_len": a.prompt_len,
                   "ctx_from": main_point["ctx"][0], "ctx_to": main_point["ctx"][1], "page_size": 16,
                   "parallelism": "none"},
        "prefill": prefill,
        "roofline": {"bound": "hbm", "achieved": round(main_point["gbs"], 1), "peak": PEAK_HBM_GBS,
                     "unit": "GB/s", "frac": round(main_point["gbs"] / PEAK_HBM_GBS, 4)},
        "points": points,
        "roofline_points": fracs,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
