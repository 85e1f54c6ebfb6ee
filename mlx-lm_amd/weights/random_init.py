"""Write a model folder (config.json, model.safetensors) with random weights."""

import json
import os


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


def main(argv=None):
    """``python -m mlx_lm_amd random_weights --config config.json --seed 2 --out DIR``."""
    import argparse

    p = argparse.ArgumentParser(prog="mlx_lm_amd random_weights",
                                description="Write a model folder with seeded random weights.")
    p.add_argument("--config", required=True, help="a config.json (its model_type chooses the architecture)")
    p.add_argument("--seed", type=int, required=True)
    p.add_argument("--out", required=True, help="folder to write config.json and model.safetensors into")
    p.add_argument("--scheme", choices=["a", "b"], default="a",
                   help="a: biases 0, norm scale 1; b: random biases and norm scales")
    p.add_argument("--dtype", choices=["float32", "bfloat16"], default="float32")
    a = p.parse_args(argv)
    with open(a.config) as fh:
        config = json.load(fh)
    write_model_folder(a.out, config, a.seed, a.scheme, a.dtype)
    print(a.out)
    return 0
