"""``python -m mlx_lm_amd <subcommand>`` in the manner of mlx_lm/cli.py:7-53."""

import importlib
import sys

from . import __version__

SUBCOMMANDS = {
    "generate": ("mlx_lm_amd.generate", "main"),
    "cache_prompt": ("mlx_lm_amd.cache_prompt", "main"),
    "trace_run": ("mlx_lm_amd.engine.replay", "main"),
    "random_weights": ("mlx_lm_amd.weights.random_init", "main"),
}


def main():
    if len(sys.argv) < 2 or sys.argv[1] in ("-h", "--help"):
        print("usage: mlx_lm_amd <subcommand> [options]\nsubcommands: " + ", ".join(sorted(SUBCOMMANDS)))
        raise SystemExit(0 if len(sys.argv) >= 2 else 1)
    if sys.argv[1] == "--version":
        print(__version__)
        return
    sub = sys.argv.pop(1)
    if sub not in SUBCOMMANDS:
        raise SystemExit(f"mlx_lm_amd: unknown subcommand '{sub}' (known: {', '.join(sorted(SUBCOMMANDS))})")
    module, fn = SUBCOMMANDS[sub]
    sys.argv[0] = f"mlx_lm_amd {sub}"
    result = getattr(importlib.import_module(module), fn)()
    if isinstance(result, int):
        raise SystemExit(result)
