"""GPT-2 inference engine for one AMD MI355X, in the manner of mlx-lm.

``load``, ``generate``, ``stream_generate`` and ``batch_generate`` are the
Python entry points (cf. mlx_lm/__init__.py:9-20).
"""

__version__ = "0.1.0"

from .generate import BatchGenerator, batch_generate, generate, generate_step, stream_generate
from .prompt_cache import (PromptCache, can_trim_prompt_cache, load_prompt_cache, make_prompt_cache,
                           save_prompt_cache, trim_prompt_cache)
from .sample_utils import make_logits_processors, make_sampler
from .utils import load

__all__ = [
    "BatchGenerator",
    "batch_generate",
    "generate",
    "generate_step",
    "stream_generate",
    "make_logits_processors",
    "make_sampler",
    "make_prompt_cache",
    "trim_prompt_cache",
    "can_trim_prompt_cache",
    "save_prompt_cache",
    "load_prompt_cache",
    "PromptCache",
    "load",
    "__version__",
]
