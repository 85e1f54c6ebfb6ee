"""Randomly drawn small GPT-2 configurations through the engine: odd widths and head sizes,
vocabularies and inner sizes that are no power of two, every page size, mixed batches with few
pages, in float32 and bfloat16, against the plain implementation and against the same requests
run whole.  The draws are fixed by their seeds."""

import random

import pytest
import torch

import helpers
import plain_gpt2 as plain
from test_engine_gpu import TOL, _plain_logits

pytestmark = pytest.mark.gpu


def _draw(seed):
    rng = random.Random(seed)
    H, hd = rng.choice([1, 2, 3, 5, 8]), rng.choice([16, 32, 48, 64, 80, 128])
    P = rng.choice([64, 130, 256, 400])
    config = dict(model_type="gpt2", n_layer=rng.randint(1, 3), n_embd=H * hd, n_head=H,
                  n_inner=rng.randint(16, 560), vocab_size=rng.randint(40, 2500), n_positions=P,
                  layer_norm_epsilon=rng.choice([1e-5, 1e-6, 1e-3]), activation_function="gelu_new")
    page_size = rng.choice([16, 32, 64])
    lengths = [min(P, rng.randint(2, P)) for _ in range(rng.randint(2, 5))]
    return config, page_size, lengths


# (seeds chosen to cover widths below a k-block of the tile kernels: n_embd 16, 32, 48)
@pytest.mark.parametrize("seed", [2, 42, 15, 57, 7, 9, 10, 16, 101, 103])
def test_random_configuration(tmp_path, seed):
    from safetensors.torch import load_file, save_file

    from mlx_lm_amd.engine import Engine, StepEntry
    from mlx_lm_amd.utils import load_model
    from mlx_lm_amd.weights import write_model_folder

    config, page_size, lengths = _draw(seed)
    folder = str(tmp_path)
    write_model_folder(folder, dict(config), seed=seed, scheme="b")
    path = folder + "/model.safetensors"
    tensors = helpers.sharpen({k: v.clone() for k, v in load_file(path).items()}, config, 3.0)
    save_file(tensors, path)
    weights = plain.from_checkpoint_layout({k: v.float() for k, v in tensors.items()}, config["n_layer"])
    tokens, steps = helpers.mixed_trace(config, seed=seed, lengths=lengths)
    held = sum(sorted(((n + 63) // 64 * 64 for n in lengths), reverse=True)[:4])
    for dtype in ("float32", "bfloat16"):
        model, _ = load_model(folder, dtype=dtype)
        eng = Engine(model, dtype=dtype, page_size=page_size, n_pages=held // page_size, max_requests=8)
        got = {rid: [] for rid in tokens}
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
            for rid in s["end"]:
                eng.end_request(rid)
            eng.cache.check()
        whole = Engine(model, dtype=dtype, page_size=page_size, n_pages=held // page_size, max_requests=8)
        for rid, toks in tokens.items():
            want = _plain_logits(weights, config, toks, dtype)
            mixed = torch.cat(got[rid]).double().cpu()
            whole.add_request(rid)
            alone = whole.step([StepEntry(rid, toks, list(range(len(toks))))]).double().cpu()
            whole.end_request(rid)
            scale = want.abs().max().item()
            what = f"seed {seed} {dtype} {config} page {page_size} lengths {lengths} request {rid}"
            assert (mixed - want).abs().max().item() <= TOL[dtype] * scale, what
            assert (alone - want).abs().max().item() <= TOL[dtype] * scale, what
            assert (mixed - alone).abs().max().item() <= TOL[dtype] * scale, what
