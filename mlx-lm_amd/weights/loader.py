"""Read safetensors files and hand a model the tensors it expects."""

import glob
import os

import torch

_DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


class WeightError(ValueError):
    """The tensors of a model folder do not match what the model expects."""


def read_safetensors(model_path):
    """All tensors of ``model*.safetensors`` in the folder, later files winning.

    mlx_lm/utils.py:336-343; no file at all is a ``FileNotFoundError`` as there.
    """
    from safetensors.torch import load_file

    files = sorted(glob.glob(os.path.join(model_path, "model*.safetensors")))
    if not files:
        raise FileNotFoundError(f"No safetensors found in {model_path}")
    tensors = {}
    for f in files:
        tensors.update(load_file(f, device="cpu"))
    return tensors


def resolve_dtype(dtype):
    if isinstance(dtype, torch.dtype):
        if dtype not in _DTYPES.values():
            raise ValueError(f"dtype {dtype} is not supported (float32 or bfloat16)")
        return dtype
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise ValueError(f"dtype '{dtype}' is not supported (float32 or bfloat16)") from None


def check_tensors(expected, tensors):
    """Raise one ``WeightError`` that lists every missing, unexpected and misshapen tensor.

    The strict load of the reference (``model.load_weights(..., strict=True)``,
    mlx_lm/utils.py:445) stops at the first offence; this names them all.
    """
    missing = sorted(n for n in expected if n not in tensors)
    unexpected = sorted(n for n in tensors if n not in expected)
    wrong = []
    for name, spec in expected.items():
        if name in tensors and tuple(tensors[name].shape) != tuple(spec.shape):
            wrong.append(f"{name}: expected {list(spec.shape)}, found {list(tensors[name].shape)}")
    bad_type = []
    for name, spec in expected.items():
        if name not in tensors:
            continue
        t = tensors[name]
        if spec.role == "int" and t.dtype.is_floating_point:
            bad_type.append(f"{name}: expected an integer table, found {t.dtype}")
        if spec.role != "int" and not t.dtype.is_floating_point:
            bad_type.append(f"{name}: expected floating point, found {t.dtype}")
    if missing or unexpected or wrong or bad_type:
        lines = ["weights do not match the model:"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        if wrong:
            lines.append(f"  wrong shape ({len(wrong)}): " + "; ".join(sorted(wrong)))
        if bad_type:
            lines.append(f"  wrong type ({len(bad_type)}): " + "; ".join(sorted(bad_type)))
        raise WeightError("\n".join(lines))


def place_tensors(expected, tensors, dtype, device):
    """Check ``tensors`` against ``expected`` and put them on ``device``.

    Matrices and tables of floats take the compute ``dtype`` (bfloat16 for
    serving, float32 for the 32-bit path); vectors (biases, norm scales and
    shifts) are kept in float32 whatever the file holds, which is exact for
    both; integer tables become int32.
    """
    dtype = resolve_dtype(dtype)
    check_tensors(expected, tensors)
    placed = {}
    for name, spec in expected.items():
        t = tensors[name]
        if spec.role == "matrix":
            t = t.to(dtype)
        elif spec.role == "vector":
            t = t.to(torch.float32)
        elif spec.role == "int":
            t = t.to(torch.int32)
        else:
            raise ValueError(f"tensor '{name}' has unknown role '{spec.role}'")
        placed[name] = t.contiguous().to(device)
    return placed
