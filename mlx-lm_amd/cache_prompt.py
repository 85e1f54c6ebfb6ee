"""``python -m mlx_lm_amd cache_prompt``: read a prompt once and save the cache it leaves.

The counterpart of mlx_lm/cache_prompt.py:19-153 (its options that this engine has, with their
names and meanings): the file it writes is what ``generate --prompt-cache-file`` goes on from.
"""

import argparse
import json
import sys
import time

from .generate import DEFAULT_PROMPT, IdTokenizer, _model_of, _peak_memory_gb, generate_step
from .prompt_cache import make_prompt_cache, save_prompt_cache

_OPTIONS = [
    (("--model",), str, None, "A local model folder (config.json, model.safetensors); not needed with --random-weights.", {}),
    (("--prompt-cache-file",), str, None, "The file to save the prompt cache in", {"required": True}),
    (("--prompt",), None, DEFAULT_PROMPT, "Message to be processed by the model ('-' reads from stdin)", {}),
    (("--prompt-ids",), str, None, "The prompt as token ids, separated by commas or spaces "
                                   "(for model folders without a tokenizer).", {}),
    # this engine's own
    (("--dtype",), None, "bfloat16", "Precision of the weights and the arithmetic.", {"choices": ["bfloat16", "float32"]}),
    (("--prefill-step-size",), int, 2048, "The most tokens of the prompt that one step reads.", {}),
    (("--random-weights",), int, None, "Draw the weights with this seed for the configuration given by --config "
                                      "(or by --model's config.json) instead of reading them.", {"metavar": "SEED"}),
    (("--config",), str, None, "A config.json for --random-weights.", {}),
]


def setup_arg_parser():
    parser = argparse.ArgumentParser(description="Cache the state of a prompt to be reused with mlx_lm_amd generate")
    for flags, kind, default, text, more in _OPTIONS:
        options = dict(default=default, help=text, **more)
        if kind is not None:
            options["type"] = kind
        parser.add_argument(*flags, **options)
    return parser


def main(argv=None):
    args = setup_arg_parser().parse_args(argv)
    model, tokenizer = _model_of(args)
    tokenizer = tokenizer if tokenizer is not None else IdTokenizer()
    if args.prompt_ids is not None:
        prompt = [int(t) for t in args.prompt_ids.replace(",", " ").split()]
    else:
        text = sys.stdin.read() if args.prompt == "-" else args.prompt
        if getattr(tokenizer, "has_chat_template", False):
            # the user's turn, left open: what follows in a later call goes on inside it
            prompt = tokenizer.apply_chat_template([{"role": "user", "content": text}], tokenize=True,
                                                   add_generation_prompt=False, continue_final_message=True)
        else:
            prompt = tokenizer.encode(text)
    cache = make_prompt_cache(model)
    start = time.time()
    widest = 0

    def progress(processed, total):
        nonlocal widest
        line = f"\rProcessed {processed:6d} tokens ({processed / max(time.time() - start, 1e-9):6.2f} tok/s)"
        widest = max(widest, len(line))
        print(line + " " * (widest - len(line)), end="", flush=True)

    for _ in generate_step(prompt, model, max_tokens=0, prompt_cache=cache, prefill_step_size=args.prefill_step_size,
                           prompt_progress_callback=progress):
        pass
    print()
    print(f"Peak memory: {_peak_memory_gb():.3f} GB")
    print("Saving...")
    save_prompt_cache(args.prompt_cache_file, cache, {"model": args.model or "", "tokenizer_config": json.dumps({})})
    return 0


if __name__ == "__main__":
    print("Calling `python -m mlx_lm_amd.cache_prompt...` directly is deprecated."
          " Use `python -m mlx_lm_amd cache_prompt ...` instead.", file=sys.stderr)
    main()
