"""Shared by the tests: tiny configurations, model folders, traces."""

import json
import os

import torch

import plain_gpt2 as plain

# Two tiny GPT-2 configurations that differ in every size and option, and a
# third with sizes that are no powers of two anywhere.
TINY_A = dict(model_type="gpt2", n_layer=2, n_embd=64, n_head=4, n_inner=256, vocab_size=512,
              n_positions=128, n_ctx=128, layer_norm_epsilon=1e-5, activation_function="gelu_new")
TINY_B = dict(model_type="gpt2", n_layer=3, n_embd=96, n_head=3, n_inner=384, vocab_size=1000,
              n_positions=256, n_ctx=256, layer_norm_epsilon=1e-6, activation_function="gelu_new")
TINY_C = dict(model_type="gpt2", n_layer=2, n_embd=240, n_head=5, n_inner=200, vocab_size=333,
              n_positions=448, layer_norm_epsilon=3e-4, activation_function="gelu_pytorch_tanh")

# Small layers and thousands of positions: a decoded row's keys are split over blocks.
TINY_LONG = dict(model_type="gpt2", n_layer=2, n_embd=64, n_head=2, n_inner=96, vocab_size=300,
                 n_positions=3400, layer_norm_epsilon=1e-5, activation_function="gelu_new")

TINY = {"A": (TINY_A, 0, "a"), "B": (TINY_B, 1, "b"), "C": (TINY_C, 5, "b"), "LONG": (TINY_LONG, 9, "a")}


def sharpen(tensors, config, score_std):
    """Scale every layer's query and key projections so that attention is
    peaked: scores get a spread of about ``score_std`` (weights drawn with
    std 0.02 give 0.0004 * n_embd), so a key that is dropped, doubled or taken
    from a wrong page changes the output by far more than rounding."""
    D = config["n_embd"]
    factor = (score_std / (0.0004 * D)) ** 0.5
    for i in range(config["n_layer"]):
        w = tensors[f"h.{i}.attn.c_attn.weight"]  # Conv1D layout [in, 3D]
        w[:, : 2 * D] *= factor
        tensors[f"h.{i}.attn.c_attn.bias"][: 2 * D] *= factor
    return tensors


def make_folder(path, name, sharp=0.0, dtype="float32"):
    """Write tiny model ``name`` to ``path``; returns (config, plain-layout float32 weights)."""
    from safetensors.torch import load_file, save_file

    from mlx_lm_amd.weights import write_model_folder

    config, seed, scheme = TINY[name]
    write_model_folder(path, dict(config), seed, scheme, dtype=dtype)
    f = os.path.join(path, "model.safetensors")
    tensors = load_file(f)
    if sharp:
        tensors = sharpen({k: v.clone() for k, v in tensors.items()}, config, sharp)
        save_file(tensors, f)
    weights = plain.from_checkpoint_layout({k: v.float() for k, v in tensors.items()}, config["n_layer"])
    return config, weights


def round_matrices_to_bf16(weights):
    """What the engine's bfloat16 path holds: matrices rounded, vectors as they are."""
    out = {}
    for k, v in weights.items():
        out[k] = v.to(torch.bfloat16).float() if v.dim() >= 2 else v
    return out


def random_tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def write_trace(path, steps):
    with open(path, "w") as fh:
        for s in steps:
            fh.write(json.dumps(s) + "\n")


def cuts_changing(n):
    sizes, out, i = [7, 2, 64, 3, 16, 2, 33, 5], [], 0
    while n > 0:
        s = min(sizes[i % len(sizes)], n)
        if n - s == 1:  # never leave a single token for the end: portions go down to two
            s += 1
        out.append(s)
        n -= s
        i += 1
    return out


def mixed_trace(config, seed, lengths, n_live=4):
    """Steps that mix portions of some requests with decoded tokens of others.

    Requests start when a place is free, run a few portions of changing size,
    then go on token by token; ends of requests give pages back for the next.
    """
    g = torch.Generator().manual_seed(seed)
    tokens = {f"r{i}": random_tokens(n, config["vocab_size"], seed * 100 + i) for i, n in enumerate(lengths)}
    waiting = list(tokens)
    live, fed, steps, step_no = [], {}, [], 0
    while waiting or live:
        while waiting and len(live) < n_live:
            rid = waiting.pop(0)
            live.append(rid)
            fed[rid] = 0
        entries, ended = [], []
        for rid in list(live):
            left = len(tokens[rid]) - fed[rid]
            if torch.rand((), generator=g).item() < 0.15 and len(live) > 1:
                continue  # left out of this step, goes on later
            prompt_part = int(len(tokens[rid]) * 0.6)
            if fed[rid] < prompt_part:
                n = int(torch.randint(2, 40, (), generator=g))
                n = min(n, prompt_part - fed[rid])
                if prompt_part - fed[rid] - n == 1:
                    n += 1
            else:
                n = 1
            n = min(n, left)
            part = tokens[rid][fed[rid] : fed[rid] + n]
            entries.append({"id": rid, "tokens": part, "want": list(range(n))})
            fed[rid] += n
            if fed[rid] == len(tokens[rid]):
                ended.append(rid)
                live.remove(rid)
        if entries:
            steps.append({"step": step_no, "entries": entries, "end": ended})
            step_no += 1
    return tokens, steps


def held(lengths, n_live):
    return sum(sorted(((n + 63) // 64 * 64 for n in lengths), reverse=True)[:n_live])


def decode_graphs(engine, n_requests):
    """The engine's recorded decode steps of ``n_requests`` requests (one a class of length)."""
    return [g for (n, _), g in engine._graphs.items() if n == n_requests]
