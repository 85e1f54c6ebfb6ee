"""Loading: config.json, the registry, weights, the tokenizer."""

import json
import os

from .config.registry import get_model_classes as _default_model_classes
from .weights.loader import place_tensors, read_safetensors, resolve_dtype


def load_config(model_path):
    """``config.json`` as a dict; ``generation_config.json`` may override ``eos_token_id``.

    mlx_lm/utils.py:277-293.
    """
    path = os.path.join(model_path, "config.json")
    try:
        with open(path) as fh:
            config = json.load(fh)
    except FileNotFoundError:
        raise FileNotFoundError(f"Config file not found in {model_path}") from None
    gen = os.path.join(model_path, "generation_config.json")
    if os.path.exists(gen):
        try:
            with open(gen) as fh:
                g = json.load(fh)
        except json.JSONDecodeError:
            g = {}
        if g.get("eos_token_id") is not None:
            config["eos_token_id"] = g["eos_token_id"]
    return config


def load_model(model_path, dtype="bfloat16", device="cuda:0", model_config=None,
               get_model_classes=_default_model_classes):
    """Build the model that ``config.json`` names and give it the folder's weights.

    The steps of mlx_lm/utils.py:296-450 that apply here: read the config
    (with overrides), look the architecture up, make its typed arguments and
    the model, read every ``model*.safetensors``, ``sanitize``, load strictly.
    Returns ``(model, config)``; the model's tensors are on ``device`` in
    ``dtype``.
    """
    config = load_config(model_path)
    if model_config:
        config.update(model_config)
    return model_from_tensors(config, read_safetensors(model_path), dtype, device, get_model_classes), config


def model_from_tensors(config, weights, dtype="bfloat16", device="cuda:0",
                       get_model_classes=_default_model_classes):
    """The model that ``config`` names, given ``weights`` under a checkpoint's names: look the
    architecture up, make its typed arguments and the model, ``sanitize``, load strictly (one
    error that lists every missing, unexpected and misshapen tensor), set dtype and device.
    What ``load_model`` does after reading the folder; callers that make their weights
    themselves (a benchmark's random ones) come in here."""
    model_cls, args_cls = get_model_classes(config)
    args = args_cls.from_dict(config)
    model = model_cls(args)
    if hasattr(model, "sanitize"):
        weights = model.sanitize(weights)
    placed = place_tensors(model.decoder.expected_tensors(), weights, dtype, device)
    model.decoder.load_tensors(placed)
    model.dtype = resolve_dtype(dtype)
    model.device = device
    return model


def load_tokenizer(model_path, eos_token_ids=None):
    """The folder's tokenizer, or ``None`` if it has none (random-weight folders)."""
    from .tokenizer_utils import load_tokenizer as _load

    return _load(model_path, eos_token_ids)


def load(path_or_hf_repo, tokenizer_config=None, model_config=None, adapter_path=None, lazy=False,
         return_config=False, revision=None, trust_remote_code=False, dtype="bfloat16",
         device="cuda:0"):
    """``(model, tokenizer)`` from a local model folder (mlx_lm/utils.py:483-541).

    Only local folders are read; adapters, remote code and lazy loading do not
    exist here and are refused rather than ignored.
    """
    if adapter_path is not None:
        raise ValueError("adapters are not supported")
    if trust_remote_code:
        raise ValueError("remote code is not supported")
    if not os.path.isdir(path_or_hf_repo):
        raise FileNotFoundError(
            f"{path_or_hf_repo} is not a local model folder (nothing is downloaded here)"
        )
    model, config = load_model(path_or_hf_repo, dtype=dtype, device=device, model_config=model_config)
    tokenizer = load_tokenizer(path_or_hf_repo, eos_token_ids=config.get("eos_token_id"))
    if return_config:
        return model, tokenizer, config
    return model, tokenizer
