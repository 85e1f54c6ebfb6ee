"""From ``model_type`` to the architecture's model and argument classes."""

import importlib

# aliases, in the manner of mlx_lm/utils.py:46-57; none is needed for GPT-2
MODEL_REMAPPING = {}

_REGISTRY = {}
_BUILTIN = {"gpt2": "mlx_lm_amd.models.gpt2"}


def register_model(model_type, model_cls, args_cls):
    """Make ``model_type`` known; later registrations replace earlier ones."""
    _REGISTRY[model_type] = (model_cls, args_cls)


def registered_model_types():
    return sorted(set(_REGISTRY) | set(_BUILTIN))


def get_model_classes(config):
    """``(Model, ModelArgs)`` for ``config["model_type"]``.

    Follows mlx_lm/utils.py:177-195: aliases first, then the architecture's
    module; an unknown type is a ``ValueError`` with the reference's text.
    """
    model_type = config.get("model_type")
    model_type = MODEL_REMAPPING.get(model_type, model_type)
    if model_type in _REGISTRY:
        return _REGISTRY[model_type]
    module = _BUILTIN.get(model_type)
    if module is None:
        raise ValueError(f"Model type {model_type} not supported.")
    arch = importlib.import_module(module)
    return arch.Model, arch.ModelArgs
