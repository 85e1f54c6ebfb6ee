"""Configuration, registry, sanitize and the weight loader's errors (no GPU)."""

import json
import os

import pytest
import torch

import helpers
from mlx_lm_amd.config import BaseModelArgs, get_model_classes, register_model
from mlx_lm_amd.models.gpt2 import Model, ModelArgs
from mlx_lm_amd.utils import load_config
from mlx_lm_amd.weights import WeightError, read_safetensors, write_model_folder
from mlx_lm_amd.weights.loader import check_tensors, place_tensors


def test_from_dict_keeps_known_keys_and_fills_defaults():
    cfg = dict(helpers.TINY_B, dropout=0.1, junk="x")
    del cfg["n_inner"]
    args = ModelArgs.from_dict(cfg)
    assert args.n_inner == 4 * args.n_embd and args.num_key_value_heads == args.n_head
    assert args.n_ctx == 256 and args.head_dim == 32 and not hasattr(args, "junk")
    cfg = dict(helpers.TINY_C)
    assert ModelArgs.from_dict(cfg).n_ctx == cfg["n_positions"]


@pytest.mark.parametrize("change,match", [
    (dict(n_head=5), "divisible"),
    (dict(activation_function="relu"), "not implemented"),
    (dict(tie_word_embeddings=False), "untied"),
    (dict(scale_attn_by_inverse_layer_idx=True), "scale_attn"),
    (dict(vocab_size=0), "positive"),
    (dict(n_embd=24, n_head=3), "head_dim"),
])
def test_what_the_engine_cannot_run_is_refused(change, match):
    cfg = dict(helpers.TINY_A, **change)
    with pytest.raises(ValueError, match=match):
        Model(ModelArgs.from_dict(cfg))


def test_num_key_value_heads_is_read_and_not_used():
    # mlx_lm/models/gpt2.py:24-26,57-58: the key is kept, keys and values are shaped with n_head
    args = ModelArgs.from_dict(dict(helpers.TINY_A, num_key_value_heads=1))
    assert args.num_key_value_heads == 1
    mixer = Model.plan(args).layers[0].parts["mixer"]
    assert mixer.params["n_kv_heads"] == mixer.params["n_heads"] == args.n_head


def test_missing_required_key_is_an_error():
    cfg = dict(helpers.TINY_A)
    del cfg["layer_norm_epsilon"]
    with pytest.raises(TypeError):
        ModelArgs.from_dict(cfg)


def test_registry():
    m, a = get_model_classes({"model_type": "gpt2"})
    assert m is Model and a is ModelArgs
    with pytest.raises(ValueError, match="Model type llama9 not supported."):
        get_model_classes({"model_type": "llama9"})

    class MyArgs(BaseModelArgs):
        pass

    class MyModel:
        pass

    register_model("my_arch", MyModel, MyArgs)
    assert get_model_classes({"model_type": "my_arch"}) == (MyModel, MyArgs)


def test_plan_names_every_size_from_the_config():
    for name in ("A", "B", "C"):
        cfg = helpers.TINY[name][0]
        model = Model(ModelArgs.from_dict(cfg))
        dec = model.decoder
        assert len(model.layers) == cfg["n_layer"] and model.model_type == "gpt2"
        assert [r.layer for r in dec.schedule] == list(range(cfg["n_layer"]))
        attn = dec.layers[0].mixer
        assert (attn.n_heads, attn.head_dim, attn.window) == (cfg["n_head"], cfg["n_embd"] // cfg["n_head"], 0)
        assert attn.scale == pytest.approx((cfg["n_embd"] // cfg["n_head"]) ** -0.5)
        assert dec.layers[0].ffn.inner == cfg["n_inner"]
        assert dec.layers[0].mixer_norm.eps == cfg["layer_norm_epsilon"] == dec.final_norm.eps
        want = dec.expected_tensors()
        assert want["model.wte.weight"].shape == (cfg["vocab_size"], cfg["n_embd"])
        assert want["model.wpe.weight"].shape == (cfg["n_positions"], cfg["n_embd"])
        assert want["model.h.0.attn.c_attn.weight"].shape == (3 * cfg["n_embd"], cfg["n_embd"])
        assert want["model.h.0.mlp.c_proj.weight"].shape == (cfg["n_embd"], cfg["n_inner"])
        assert want["model.ln_f.bias"].role == "vector"
        assert len(want) == 2 + 12 * cfg["n_layer"] + 2  # the tied head adds no tensor
        needs = dec.cache_needs()
        assert len(needs) == cfg["n_layer"] and needs[0].n_kv_heads == cfg["n_head"]


def test_sanitize_matches_the_plain_conversion(tmp_path):
    cfg, weights = helpers.make_folder(str(tmp_path), "B")
    model = Model(ModelArgs.from_dict(cfg))
    raw = read_safetensors(str(tmp_path))
    assert raw["h.0.attn.c_attn.weight"].shape == (cfg["n_embd"], 3 * cfg["n_embd"])  # Conv1D layout
    raw["h.1.attn.bias"] = torch.ones(1, 1, 4, 4)
    raw["h.1.attn.masked_bias"] = torch.tensor(-1e4)
    raw = {"transformer." + k: v for k, v in raw.items()}
    raw["lm_head.weight"] = raw["transformer.wte.weight"].clone()
    clean = model.sanitize(raw)
    assert set(clean) == set(weights)
    for k in weights:
        assert torch.equal(clean[k], weights[k]), k
    # sanitizing again changes nothing: prefixed names are not transposed twice
    again = model.sanitize(dict(clean))
    assert all(torch.equal(again[k], clean[k]) for k in clean)
    check_tensors(model.decoder.expected_tensors(), clean)
    raw["lm_head.weight"] = raw["lm_head.weight"] + 1
    with pytest.raises(ValueError, match="tied"):
        model.sanitize(raw)


def test_one_error_lists_missing_unexpected_and_misshapen():
    cfg = helpers.TINY_A
    model = Model(ModelArgs.from_dict(cfg))
    t = model.sanitize(Model.random_weights(model.args, 0))
    del t["model.h.1.ln_2.bias"]
    del t["model.wpe.weight"]
    t["model.h.7.extra"] = torch.zeros(3)
    t["model.ln_f.weight"] = torch.zeros(cfg["n_embd"] + 1)
    t["model.h.0.mlp.c_fc.weight"] = t["model.h.0.mlp.c_fc.weight"].t().contiguous()
    with pytest.raises(WeightError) as e:
        check_tensors(model.decoder.expected_tensors(), t)
    msg = str(e.value)
    assert "missing (2): model.h.1.ln_2.bias, model.wpe.weight" in msg
    assert "unexpected (1): model.h.7.extra" in msg
    assert "model.ln_f.weight: expected [64], found [65]" in msg
    assert "model.h.0.mlp.c_fc.weight: expected [256, 64], found [64, 256]" in msg


def test_placement_dtypes():
    cfg = helpers.TINY_A
    model = Model(ModelArgs.from_dict(cfg))
    t = model.sanitize(Model.random_weights(model.args, 0, "b"))
    placed = place_tensors(model.decoder.expected_tensors(), t, "bfloat16", "cpu")
    assert placed["model.wte.weight"].dtype == torch.bfloat16
    assert placed["model.h.0.attn.c_attn.weight"].dtype == torch.bfloat16
    assert placed["model.h.0.attn.c_attn.bias"].dtype == torch.float32  # stays 32-bit
    assert placed["model.ln_f.weight"].dtype == torch.float32
    assert torch.equal(placed["model.ln_f.weight"], t["model.ln_f.weight"])
    placed = place_tensors(model.decoder.expected_tensors(), t, "float32", "cpu")
    assert all(v.dtype == torch.float32 for v in placed.values())
    with pytest.raises(ValueError, match="not supported"):
        place_tensors(model.decoder.expected_tensors(), t, "float16", "cpu")


def test_random_model_folder_is_seeded_and_complete(tmp_path):
    a, b, c = (str(tmp_path / n) for n in "abc")
    write_model_folder(a, dict(helpers.TINY_A), 0, "a")
    write_model_folder(b, dict(helpers.TINY_A), 0, "a")
    write_model_folder(c, dict(helpers.TINY_A), 1, "b")
    assert sorted(os.listdir(a)) == ["config.json", "model.safetensors"]
    assert load_config(a) == helpers.TINY_A
    ta, tb, tc = read_safetensors(a), read_safetensors(b), read_safetensors(c)
    assert all(torch.equal(ta[k], tb[k]) for k in ta)
    assert not torch.equal(ta["wte.weight"], tc["wte.weight"])
    # scheme a: biases 0, scales 1; scheme b: neither
    assert ta["h.0.ln_1.weight"].eq(1).all() and ta["h.1.mlp.c_fc.bias"].eq(0).all()
    assert not tc["h.0.ln_1.weight"].eq(1).any() and tc["h.1.mlp.c_fc.bias"].abs().sum() > 0
    L = helpers.TINY_A["n_layer"]
    assert abs(ta["wte.weight"].std().item() - 0.02) < 1e-3
    assert abs(ta["h.0.mlp.c_proj.weight"].std().item() - 0.02 / (2 * L) ** 0.5) < 1e-3
    with pytest.raises(FileNotFoundError, match="No safetensors found"):
        read_safetensors(str(tmp_path))
    with pytest.raises(FileNotFoundError):
        load_config(str(tmp_path))


def test_generation_config_overrides_eos(tmp_path):
    d = str(tmp_path)
    json.dump(dict(helpers.TINY_A, eos_token_id=5), open(os.path.join(d, "config.json"), "w"))
    json.dump({"eos_token_id": [7, 8]}, open(os.path.join(d, "generation_config.json"), "w"))
    assert load_config(d)["eos_token_id"] == [7, 8]


def test_plan_validation():
    from mlx_lm_amd.config import RunEntry

    plan = Model.plan(ModelArgs.from_dict(helpers.TINY_A))
    plan.schedule = [RunEntry(0, 0), RunEntry(1, 1), RunEntry(0, 2), RunEntry(1, 1, writes_cache=False)]
    assert plan.validate().n_cache_slots == 3
    plan.schedule = [RunEntry(0, 0), RunEntry(1, 0)]
    with pytest.raises(ValueError, match="written twice"):
        plan.validate()
    plan.schedule = [RunEntry(0, 1, writes_cache=False), RunEntry(1, 1)]
    with pytest.raises(ValueError, match="before any run"):
        plan.validate()
    plan.schedule = [RunEntry(5, 0)]
    with pytest.raises(ValueError, match="names layer 5"):
        plan.validate()


def test_random_weights_from_the_command_line(tmp_path):
    """``python -m mlx_lm_amd random_weights`` writes the folder that the function writes."""
    import json
    import subprocess
    import sys

    from safetensors.torch import load_file

    from mlx_lm_amd.weights import write_model_folder

    config = dict(model_type="gpt2", n_layer=2, n_embd=48, n_head=3, n_positions=40, vocab_size=77,
                  layer_norm_epsilon=1e-6, n_inner=100)
    cfg = tmp_path / "c.json"
    cfg.write_text(json.dumps(config))
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-m", "mlx_lm_amd", "random_weights", "--config", str(cfg), "--seed", "5",
                        "--scheme", "b", "--out", str(tmp_path / "cli")], cwd=root, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    write_model_folder(str(tmp_path / "fn"), config, 5, "b")
    a, b = load_file(str(tmp_path / "cli" / "model.safetensors")), load_file(str(tmp_path / "fn" / "model.safetensors"))
    assert sorted(a) == sorted(b) and all(torch.equal(a[k], b[k]) for k in a)
    assert json.loads((tmp_path / "cli" / "config.json").read_text()) == config


def test_weights_cannot_be_swapped_under_a_model_that_has_run():
    """The native twins of the parts (and the steps an engine recorded) hold the addresses of the
    weights they were made from: a second load would leave them reading the old tensors."""
    model = Model(ModelArgs.from_dict(helpers.TINY_A))
    t = model.sanitize(Model.random_weights(model.args, 0, "a"))
    placed = place_tensors(model.decoder.expected_tensors(), t, "float32", "cpu")
    model.decoder.load_tensors(placed)
    model.decoder.load_tensors(placed)  # nothing has been made from them yet: fine
    part = model.decoder.final_norm
    part._native = 1  # (stands for a twin; never handed to the library)
    try:
        with pytest.raises(RuntimeError, match="build a new model"):
            model.decoder.load_tensors(placed)
    finally:
        part._native = None
