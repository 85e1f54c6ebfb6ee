"""Write a model folder (config.json, model.safetensors) with random weights."""

import json
import os

import torch

from ..config.registry import get_model_classes


def write_model_folder(path, config, seed, scheme="a", dtype="float32", get_model_classes=get_model_classes):
    """Make ``path`` a model folder for ``config`` (the dict of config.json).

    The architecture named by ``config["model_type"]`` draws the tensors
    (its ``random_weights``), in the names and layouts of its checkpoints, so
    loading the folder goes through the same ``sanitize`` as a real one.
    """
    from safetensors.torch import save_file

    from .loader import resolve_dtype

    model_cls, args_cls = get_model_classes(config)
    args = args_cls.from_dict(config)
    tensors = model_cls.random_weights(args, seed, scheme)
    dt = resolve_dtype(dtype)
    tensors = {
        k: (v.to(dt) if v.dtype.is_floating_point else v).contiguous() for k, v in tensors.items()
    }
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as fh:
        json.dump(config, fh, indent=1)
    save_file(tensors, os.path.join(path, "model.safetensors"))
    return path
