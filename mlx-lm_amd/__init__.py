"""GPT-2 inference engine for one AMD MI355X, in the manner of mlx-lm.

``load``, ``generate``, ``stream_generate`` and ``batch_generate`` are the
Python entry points (cf. mlx_lm/__init__.py:9-20); they are imported at first
use so that tools which only need a part of the package stay light.
"""

__version__ = "0.1.0"

_LAZY = {
    "load": ("utils", "load"),
    "generate": ("generate", "generate"),
    "stream_generate": ("generate", "stream_generate"),
    "batch_generate": ("generate", "batch_generate"),
    "generate_step": ("generate", "generate_step"),
    "BatchGenerator": ("generate", "BatchGenerator"),
    "make_sampler": ("sample_utils", "make_sampler"),
    "make_logits_processors": ("sample_utils", "make_logits_processors"),
}

__all__ = sorted(_LAZY) + ["__version__"]


def __getattr__(name):
    if name in _LAZY:
        import importlib

        module, attr = _LAZY[name]
        return getattr(importlib.import_module(f"{__name__}.{module}"), attr)
    raise AttributeError(f"module '{__name__}' has no attribute '{name}'")
