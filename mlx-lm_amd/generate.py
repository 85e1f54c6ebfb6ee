"""Generation: ``generate_step``, ``stream_generate``, ``generate``,
``BatchGenerator``, ``batch_generate`` and the ``generate`` command line,
with the names and meanings of mlx_lm/generate.py.

All of them run on the continuous-batching scheduler and the step function of
``mlx_lm_amd.engine``; a single request is a batch of one.
"""

import argparse
import contextlib
import json
import sys
import time
from dataclasses import dataclass
from typing import Any, List, Optional

import torch

from . import sample_utils
from .engine.scheduler import Request, Scheduler
from .engine.step import Engine
from .sample_utils import Sampler, make_logits_processors, make_sampler
from .sampling import PendingRead, SamplerBuffers, apply_processors, sample_batch

DEFAULT_PROMPT = "hello"
DEFAULT_MAX_TOKENS = 100
DEFAULT_TEMP = 0.0
DEFAULT_TOP_P = 1.0
DEFAULT_MIN_P = 0.0
DEFAULT_TOP_K = 0
DEFAULT_XTC_PROBABILITY = 0.0
DEFAULT_XTC_THRESHOLD = 0.0
DEFAULT_MIN_TOKENS_TO_KEEP = 1
DEFAULT_SEED = None

_GREEDY = Sampler()


# ---------------------------------------------------------------------------
# engines are made once per model and cache geometry


def engine_for(model, page_size=16, max_requests=64, max_cache_tokens=None):
    """The model's engine; made at first use and kept on the model.

    The page pool holds ``max_cache_tokens`` tokens; by default as many as
    ``max_requests`` full contexts, but not more than 60 % of the free
    device memory.
    """
    key = (page_size, max_requests, max_cache_tokens)
    engines = model.__dict__.setdefault("_engines", {})
    eng = engines.get(key)
    if eng is None:
        dec = model.decoder
        if max_cache_tokens is None:
            from .cache import CacheManager

            probe = CacheManager(dec.cache_needs(), page_size, 1, 1, dtype=model.dtype)
            per_token = max(1, probe.bytes_per_token())
            free, _ = torch.cuda.mem_get_info(torch.device(model.device))
            max_cache_tokens = min(max_requests * dec.max_positions, int(free * 0.6) // per_token)
            max_cache_tokens = max(max_cache_tokens, dec.max_positions)
        # (a scheduler's steps keep coming back in the same shapes: portions of one size beside
        # the requests that decode; those are recorded as the decode steps are)
        eng = Engine(model, dtype=model.dtype, device=model.device, page_size=page_size,
                     max_tokens=max_cache_tokens, max_requests=max_requests, record_prompt_steps=True)
        engines[key] = eng
    return eng


class SampleJob:
    """A sampling call whose tokens are on their way to the host."""

    def __init__(self, requests, tokens, read, logprobs, custom):
        self.requests = requests
        self.tokens = tokens      # int32 device array, a row per request: what the next step can be fed
        self.read = read          # PendingRead
        self.logprobs = logprobs  # float32 [rows, vocab] on the device, or None
        self.custom = custom      # requests whose sampler is a callable: their token is made on the host
        self.feedable = not custom


class _SampleFn:
    """The scheduler's sampling callback: processors, log-probabilities, one draw per row.

    ``logits processors -> logprobs = logits - logsumexp -> sampler`` as in
    mlx_lm/generate.py:400-412,1417-1445, for all rows in one launch each.
    ``launch`` queues the work and returns at once; ``finish`` waits for the
    tokens; calling the object does both.  The arrays that tokens pass through
    are this object's own: other generators' sampling calls, however many come
    in between, leave a call's tokens alone until its scheduler has fed them on.
    """

    def __init__(self):
        self.buffers = SamplerBuffers()

    def launch(self, logits, requests):
        if any(r.logits_processors for r in requests):
            apply_processors(logits, [r.logits_processors or [] for r in requests],
                             [r.tokens for r in requests])
        samplers = [r.sampler if isinstance(r.sampler, Sampler) else _GREEDY for r in requests]
        custom = [r for r in requests if r.sampler is not None and not isinstance(r.sampler, Sampler)]
        want = bool(custom) or any(r.want_logprobs for r in requests)
        out = sample_batch(logits, samplers, [r.seed for r in requests],
                           [len(r.generated) for r in requests], want_logprobs=want, buffers=self.buffers)
        read = PendingRead(out[0], out[1], buffers=self.buffers)
        return SampleJob(list(requests), out[0], read, out[2] if want else None, custom)

    def finish(self, job):
        tokens, token_lp = job.read.wait()
        results = []
        for i, r in enumerate(job.requests):
            tok, lp = tokens[i], token_lp[i]
            if r in job.custom:  # any callable on log-probabilities, as the reference allows
                tok = int(torch.as_tensor(r.sampler(job.logprobs[i : i + 1])).reshape(-1)[0])
                lp = float(job.logprobs[i, tok])
            results.append((tok, lp, job.logprobs[i] if (job.logprobs is not None and r.want_logprobs) else None))
        return results

    def __call__(self, logits, requests):
        return self.finish(self.launch(logits, requests))


def make_sample_fn():
    return _SampleFn()


# ---------------------------------------------------------------------------
# one request


_UNSUPPORTED = {
    "max_kv_size": None, "prompt_cache": None, "kv_bits": None, "input_embeddings": None,
    "draft_model": None,
}


def _refuse_unsupported(kwargs):
    for k, default in _UNSUPPORTED.items():
        if kwargs.pop(k, default) is not None:
            raise ValueError(f"'{k}' is not supported by this engine")
    kwargs.pop("kv_group_size", None)
    kwargs.pop("quantized_kv_start", None)
    kwargs.pop("num_draft_tokens", None)


_uid = [0]


def generate_step(prompt, model, *, max_tokens=256, sampler=None, logits_processors=None,
                  prefill_step_size=2048, prompt_progress_callback=None, seed=None, **kwargs):
    """Yield ``(token, logprobs)`` for one prompt (mlx_lm/generate.py:298-461).

    The prompt is read in portions of ``prefill_step_size``; then one token
    per step.  ``logprobs`` is a float32 device tensor ``[vocab]``.  Exactly
    ``max_tokens`` tokens are yielded unless the model's positions run out.
    """
    _refuse_unsupported(kwargs)
    if kwargs:
        raise TypeError(f"unknown options: {sorted(kwargs)}")
    prompt = [int(t) for t in (prompt.tolist() if hasattr(prompt, "tolist") else prompt)]
    if len(prompt) == 0:
        raise ValueError("Either input_embeddings or prompt (or both) must be provided.")
    engine = engine_for(model)
    sched = Scheduler(engine, make_sample_fn(), max_num_seqs=1,
                      max_num_batched_tokens=prefill_step_size, prefill_step_size=prefill_step_size)
    _uid[0] += 1
    rid = ("generate_step", _uid[0])
    if seed is None:
        seed = getattr(sampler, "seed", None)
    if seed is None:
        seed = sample_utils.default_seed()
    req = Request(rid, prompt, max_tokens, sampler=sampler, logits_processors=logits_processors,
                  seed=seed, want_logprobs=True)
    sched.add(req)
    try:
        while sched.has_work:
            outs = sched.step()
            if prompt_progress_callback is not None and not req.generated:
                prompt_progress_callback(min(req.num_computed, len(prompt)), len(prompt))
            for o in outs:
                yield o.token, o.logprobs
    finally:
        if engine.has_request(rid):
            sched.abort(rid)


@dataclass
class GenerationResponse:
    """What ``stream_generate`` yields (mlx_lm/generate.py:260-287)."""

    text: str
    token: int
    logprobs: Any
    from_draft: bool
    prompt_tokens: int
    prompt_tps: float
    generation_tokens: int
    generation_tps: float
    peak_memory: float
    finish_reason: Optional[str] = None


class IdTokenizer:
    """Stands in where a model folder has no tokenizer: text is token ids in decimal."""

    bos_token = None

    def __init__(self):
        self.eos_token_ids = set()

    def add_eos_token(self, token):
        self.eos_token_ids.add(int(token))

    def encode(self, text, add_special_tokens=True):
        return [int(t) for t in text.replace(",", " ").split()]

    def decode(self, ids, skip_special_tokens=False):
        return " ".join(str(int(t)) for t in ids)

    @property
    def detokenizer(self):
        return _IdDetokenizer()


class _IdDetokenizer:
    def __init__(self):
        self.reset()

    def reset(self):
        self.tokens, self.text, self._offset = [], "", 0

    def add_token(self, token):
        self.tokens.append(int(token))
        self.text += ("" if len(self.tokens) == 1 else " ") + str(int(token))

    def finalize(self):
        pass

    @property
    def last_segment(self):
        seg = self.text[self._offset :]
        self._offset = len(self.text)
        return seg


def _peak_memory_gb():
    return torch.cuda.max_memory_allocated() / 1e9


def stream_generate(model, tokenizer, prompt, max_tokens=256, draft_model=None, **kwargs):
    """Yield a ``GenerationResponse`` per token (mlx_lm/generate.py:648-744).

    Stops at an end-of-sequence token (which is not added to the text) or
    after ``max_tokens``; the last response carries ``finish_reason``.
    """
    if draft_model is not None:
        raise ValueError("speculative decoding is not supported")
    if tokenizer is None:
        tokenizer = IdTokenizer()
    if isinstance(prompt, str):
        add_special = tokenizer.bos_token is None or not prompt.startswith(tokenizer.bos_token)
        prompt = tokenizer.encode(prompt, add_special_tokens=add_special)
    prompt = [int(t) for t in (prompt.tolist() if hasattr(prompt, "tolist") else prompt)]
    detokenizer = tokenizer.detokenizer
    kwargs["max_tokens"] = max_tokens
    tic = time.perf_counter()
    prompt_tps = 0.0
    n, token, logprobs = -1, None, None
    for n, (token, logprobs) in enumerate(generate_step(prompt, model, **kwargs)):
        if n == 0:
            prompt_time = time.perf_counter() - tic
            prompt_tps = len(prompt) / prompt_time
            tic = time.perf_counter()
        if token in tokenizer.eos_token_ids:
            break
        detokenizer.add_token(token)
        if (n + 1) == max_tokens:
            break
        yield GenerationResponse(
            text=detokenizer.last_segment, token=token, logprobs=logprobs, from_draft=False,
            prompt_tokens=len(prompt), prompt_tps=prompt_tps, generation_tokens=n + 1,
            generation_tps=(n + 1) / max(time.perf_counter() - tic, 1e-9),
            peak_memory=_peak_memory_gb(), finish_reason=None)
    if n < 0:
        return
    detokenizer.finalize()
    yield GenerationResponse(
        text=detokenizer.last_segment, token=token, logprobs=logprobs, from_draft=False,
        prompt_tokens=len(prompt), prompt_tps=prompt_tps, generation_tokens=n + 1,
        generation_tps=(n + 1) / max(time.perf_counter() - tic, 1e-9),
        peak_memory=_peak_memory_gb(),
        finish_reason="stop" if token in tokenizer.eos_token_ids else "length")


def generate(model, tokenizer, prompt, verbose=False, **kwargs):
    """The whole response as text (mlx_lm/generate.py:747-790).

    Without a tokenizer the text is the generated token ids in decimal.
    """
    if verbose:
        print("=" * 10)
    text = ""
    response = None
    for response in stream_generate(model, tokenizer, prompt, **kwargs):
        if verbose:
            print(response.text, end="", flush=True)
        text += response.text
    if verbose:
        print()
        print("=" * 10)
        if len(text) == 0:
            print("No text generated for this prompt")
            return
        print(f"Prompt: {response.prompt_tokens} tokens, {response.prompt_tps:.3f} tokens-per-sec")
        print(f"Generation: {response.generation_tokens} tokens, "
              f"{response.generation_tps:.3f} tokens-per-sec")
        print(f"Peak memory: {response.peak_memory:.3f} GB")
    return text


# ---------------------------------------------------------------------------
# many requests


@dataclass
class BatchStats:
    """mlx_lm/generate.py:805-826."""

    prompt_tokens: int = 0
    prompt_tps: float = 0
    prompt_time: float = 0
    generation_tokens: int = 0
    generation_tps: float = 0
    generation_time: float = 0
    peak_memory: float = 0


@dataclass
class BatchResponse:
    """mlx_lm/generate.py:1948-1968."""

    texts: List[str]
    stats: BatchStats
    caches: Optional[list]
    token_ids: Optional[List[List[int]]] = None
    logprobs: Optional[List[List[float]]] = None


class BatchGenerator:
    """Continuous batching with the reference's surface (mlx_lm/generate.py:1565-1945).

    ``insert`` queues prompts and returns their uids; ``next`` runs one step
    and returns ``(prompt_responses, generation_responses)``;
    ``next_generated`` runs steps until tokens were generated or nothing is
    left; ``remove`` drops requests.  ``completion_batch_size`` bounds the
    requests that run at once, ``prefill_step_size`` a prompt's portion and
    ``prefill_batch_size * prefill_step_size`` the tokens of one step.
    """

    @dataclass
    class PromptResponse:
        uid: int
        progress: tuple
        end_of_prompt: bool

    @dataclass
    class Response:
        uid: int
        token: int
        logprobs: Any
        finish_reason: Optional[str]
        prompt_cache: Any = None
        all_tokens: Optional[List[int]] = None
        token_logprob: float = 0.0

    def __init__(self, model, *, max_tokens=128, stop_tokens=None, sampler=None,
                 logits_processors=None, completion_batch_size=32, prefill_batch_size=8,
                 prefill_step_size=2048, max_kv_size=None, stream=None, seed=None,
                 want_logprobs=True, engine=None):
        if max_kv_size is not None:
            raise ValueError("'max_kv_size' is not supported by this engine")
        self.model = model
        self.max_tokens = max_tokens
        self.sampler = sampler
        self.logits_processors = logits_processors or []
        self.stop_tokens = [list(s) for s in (stop_tokens or [])]
        self.completion_batch_size = max(completion_batch_size, prefill_batch_size)
        self.prefill_batch_size = prefill_batch_size
        self.prefill_step_size = prefill_step_size
        self.seed = sample_utils.default_seed() if seed is None else seed
        self.want_logprobs = want_logprobs
        self.engine = engine or engine_for(model, max_requests=max(64, self.completion_batch_size))
        self.scheduler = Scheduler(
            self.engine, make_sample_fn(), max_num_seqs=self.completion_batch_size,
            max_num_batched_tokens=prefill_batch_size * prefill_step_size + self.completion_batch_size,
            prefill_step_size=prefill_step_size)
        self._uid_count = 0
        self._requests = {}
        self._prompt_tokens_counter = 0
        self._prompt_time_counter = 0.0
        self._gen_tokens_counter = 0

    def close(self):
        for uid in list(self._requests):
            self.remove([uid])

    @contextlib.contextmanager
    def stats(self, stats=None):
        stats = stats or BatchStats()
        self._prompt_tokens_counter = 0
        self._prompt_time_counter = 0.0
        self._gen_tokens_counter = 0
        tic = time.perf_counter()
        try:
            yield stats
        finally:
            total = time.perf_counter() - tic
            gen_time = total - self._prompt_time_counter
            stats.prompt_tokens += self._prompt_tokens_counter
            stats.prompt_time += self._prompt_time_counter
            stats.prompt_tps = stats.prompt_tokens / max(stats.prompt_time, 1e-9)
            stats.generation_tokens += self._gen_tokens_counter
            stats.generation_time += gen_time
            stats.generation_tps = stats.generation_tokens / max(stats.generation_time, 1e-9)
            stats.peak_memory = max(stats.peak_memory, _peak_memory_gb())

    def insert(self, prompts, max_tokens=None, caches=None, all_tokens=None, samplers=None,
               logits_processors=None, stop_matchers=None, seeds=None):
        """Queue prompts; per-request lists override the generator's defaults.

        ``stop_matchers[i]`` is a list of token-id sequences that stop request
        ``i``.  ``seeds[i]`` keys its random draws (default: the generator's
        seed plus the uid).
        """
        if caches is not None and any(c is not None for c in caches):
            raise ValueError("re-inserting prompt caches is not supported")
        uids = []
        for i, p in enumerate(prompts):
            uid = self._uid_count
            self._uid_count += 1
            req = Request(
                uid, [int(t) for t in p],
                self.max_tokens if max_tokens is None else max_tokens[i],
                sampler=(samplers[i] if samplers and samplers[i] is not None else self.sampler),
                logits_processors=(logits_processors[i] if logits_processors and logits_processors[i]
                                   else self.logits_processors),
                stop_sequences=(stop_matchers[i] if stop_matchers and stop_matchers[i] is not None
                                else self.stop_tokens),
                seed=(seeds[i] if seeds else self.seed + uid),
                want_logprobs=self.want_logprobs)
            self.scheduler.add(req)
            if req.finish_reason is None:  # (a request for no tokens at all is over already)
                self._requests[uid] = req
            uids.append(uid)
        return uids

    def remove(self, uids, return_prompt_caches=False):
        for uid in uids:
            if uid in self._requests:
                try:
                    self.scheduler.abort(uid)
                except KeyError:
                    pass
                del self._requests[uid]
        return {} if return_prompt_caches else None

    def _next(self):
        before = {uid: (r.num_computed, bool(r.generated)) for uid, r in self._requests.items()}
        tic = time.perf_counter()
        outs = self.scheduler.step()
        elapsed = time.perf_counter() - tic
        prompt_responses, prompt_tokens = [], 0
        for uid, (done, had_generated) in before.items():
            r = self._requests[uid]
            if not had_generated and r.num_computed != done:
                n = min(r.num_computed, len(r.prompt)) - min(done, len(r.prompt))
                prompt_tokens += n
                prompt_responses.append(self.PromptResponse(
                    uid, (min(r.num_computed, len(r.prompt)), len(r.prompt)),
                    r.num_computed >= len(r.prompt)))
        # a step's time counts as prompt time in proportion to its prompt tokens
        total = prompt_tokens + len(outs)
        if total:
            self._prompt_time_counter += elapsed * prompt_tokens / total
        self._prompt_tokens_counter += prompt_tokens
        self._gen_tokens_counter += len(outs)
        responses = []
        for o in outs:
            r = self._requests[o.request_id]
            responses.append(self.Response(o.request_id, o.token, o.logprobs, o.finish_reason, None,
                                           r.tokens if o.finish_reason else None, o.logprob))
            if o.finish_reason is not None:
                del self._requests[o.request_id]
        return prompt_responses, responses

    def next(self):
        return self._next()

    def next_generated(self):
        while self.scheduler.has_work:
            _, responses = self._next()
            if responses:
                return responses
        return []


def batch_generate(model, tokenizer, prompts, prompt_caches=None, max_tokens=128, verbose=False,
                   return_prompt_caches=False, return_token_ids=False, return_logprobs=False,
                   **kwargs):
    """Run a list of prompts to completion (mlx_lm/generate.py:1971-2060)."""
    if prompt_caches is not None or return_prompt_caches:
        raise ValueError("prompt caches are not supported")
    if tokenizer is None:
        tokenizer = IdTokenizer()
    gen = BatchGenerator(model, stop_tokens=[[t] for t in tokenizer.eos_token_ids],
                         want_logprobs=False, **kwargs)
    num_samples, fin = len(prompts), 0
    if verbose:
        print(f"[batch_generate] Finished processing 0/{num_samples} ...", end="\r")
    if isinstance(max_tokens, int):
        max_tokens = [max_tokens] * len(prompts)
    uids = gen.insert(prompts, max_tokens)
    results = {uid: [] for uid in uids}
    logprob_results = {uid: [] for uid in uids}
    with gen.stats() as stats:
        while responses := gen.next_generated():
            for r in responses:
                if r.finish_reason is not None and verbose:
                    fin += 1
                    print(f"[batch_generate] Finished processing {fin}/{num_samples} ...", end="\r")
                if r.finish_reason != "stop":
                    results[r.uid].append(r.token)
                    logprob_results[r.uid].append(r.token_logprob)
    gen.close()
    if verbose:
        print(f"[batch_generate] Finished processing {fin}/{num_samples}")
    texts = [tokenizer.decode(results[uid]) for uid in uids]
    token_ids = [results[uid] for uid in uids] if return_token_ids else None
    logprobs = [logprob_results[uid] for uid in uids] if return_logprobs else None
    if verbose:
        print(f"[batch_generate] Prompt: {stats.prompt_tokens} tokens, {stats.prompt_tps:.3f} tokens-per-sec")
        print(f"[batch_generate] Generation: {stats.generation_tokens} tokens, "
              f"{stats.generation_tps:.3f} tokens-per-sec")
        print(f"[batch_generate] Peak memory: {stats.peak_memory:.3f} GB")
    return BatchResponse(texts, stats, None, token_ids, logprobs)


# ---------------------------------------------------------------------------
# command line


def str2bool(string):
    return string.lower() not in ["false", "f"]


def setup_arg_parser():
    """The options of ``mlx_lm.generate`` that this engine has (mlx_lm/generate.py:54-213)."""
    parser = argparse.ArgumentParser(description="LLM inference script")
    parser.add_argument("--model", type=str, required=True,
                        help="The path to the local model directory.")
    parser.add_argument("--extra-eos-token", type=str, default=(), nargs="+",
                        help="Add tokens in the list of eos tokens that stop generation.")
    parser.add_argument("--system-prompt", default=None,
                        help="System prompt to be used for the chat template")
    parser.add_argument("--prompt", "-p", default=DEFAULT_PROMPT,
                        help="Message to be processed by the model ('-' reads from stdin)")
    parser.add_argument("--prompt-ids", type=str, default=None,
                        help="The prompt as token ids separated by commas or spaces "
                        "(for model folders without a tokenizer)")
    parser.add_argument("--prefill-response", default=None,
                        help="Prefill response to be used for the chat template")
    parser.add_argument("--max-tokens", "-m", type=int, default=DEFAULT_MAX_TOKENS,
                        help="Maximum number of tokens to generate")
    parser.add_argument("--temp", type=float, default=DEFAULT_TEMP, help="Sampling temperature")
    parser.add_argument("--top-p", type=float, default=DEFAULT_TOP_P, help="Sampling top-p")
    parser.add_argument("--min-p", type=float, default=DEFAULT_MIN_P, help="Sampling min-p")
    parser.add_argument("--top-k", type=int, default=DEFAULT_TOP_K, help="Sampling top-k")
    parser.add_argument("--xtc-probability", type=float, default=DEFAULT_XTC_PROBABILITY,
                        help="Probability of XTC sampling to happen each next token")
    parser.add_argument("--xtc-threshold", type=float, default=0.1,
                        help="Threshold the probs of each next token candidate to be sampled by XTC")
    parser.add_argument("--min-tokens-to-keep", type=int, default=DEFAULT_MIN_TOKENS_TO_KEEP,
                        help="Minimum tokens to keep for min-p sampling.")
    parser.add_argument("--seed", type=int, default=DEFAULT_SEED, help="PRNG seed")
    parser.add_argument("--ignore-chat-template", action="store_true",
                        help="Use the raw prompt without the tokenizer's chat template.")
    parser.add_argument("--chat-template-config", default=None,
                        help="Additional config for `apply_chat_template`. Should be a dictionary of "
                        "string keys to values represented as a JSON decodable string.")
    parser.add_argument("--verbose", type=str2bool, default=True,
                        help="Log verbose output when 'True' or 'T' or only print the response "
                        "when 'False' or 'F'")
    parser.add_argument("--dtype", choices=["bfloat16", "float32"], default="bfloat16",
                        help="Compute precision")
    parser.add_argument("--prefill-step-size", type=int, default=2048,
                        help="Most prompt tokens read in one step")
    return parser


def chat_prompt(tokenizer, prompt, args):
    """The prompt inside the tokenizer's chat template, as token ids (mlx_lm/generate.py:2115-2152).

    A tokenizer without a template, or ``--ignore-chat-template``, leaves the text as it is.
    """
    if args.ignore_chat_template or not getattr(tokenizer, "has_chat_template", False):
        return prompt
    template_kwargs = json.loads(args.chat_template_config) if args.chat_template_config else {}
    messages = []
    if args.system_prompt is not None:
        messages.append({"role": "system", "content": args.system_prompt})
    messages.append({"role": "user", "content": prompt})
    has_prefill = args.prefill_response is not None
    if has_prefill:
        messages.append({"role": "assistant", "content": args.prefill_response})
    return tokenizer.apply_chat_template(messages, tokenize=True, continue_final_message=has_prefill,
                                         add_generation_prompt=not has_prefill, **template_kwargs)


def main(argv=None):
    parser = setup_arg_parser()
    args = parser.parse_args(argv)
    if args.seed is not None:
        sample_utils.seed(args.seed)
    from .utils import load

    model, tokenizer = load(args.model, dtype=args.dtype)
    if tokenizer is None:
        tokenizer = IdTokenizer()
    for tok in args.extra_eos_token:
        tokenizer.add_eos_token(tok)
    if args.prompt_ids is not None:
        prompt = [int(t) for t in args.prompt_ids.replace(",", " ").split()]
    else:
        prompt = args.prompt.replace("\\n", "\n").replace("\\t", "\t")
        prompt = sys.stdin.read() if prompt == "-" else prompt
        prompt = chat_prompt(tokenizer, prompt, args)
    special = []
    if args.xtc_probability > 0:  # tokens that XTC never removes (mlx_lm/generate.py:2168)
        special = list(tokenizer.encode("\n", add_special_tokens=False)) + sorted(tokenizer.eos_token_ids)
    sampler = make_sampler(args.temp, args.top_p, args.min_p, args.min_tokens_to_keep,
                           top_k=args.top_k, xtc_probability=args.xtc_probability,
                           xtc_threshold=args.xtc_threshold, xtc_special_tokens=special)
    response = generate(model, tokenizer, prompt, max_tokens=args.max_tokens, verbose=args.verbose,
                        sampler=sampler, prefill_step_size=args.prefill_step_size)
    if not args.verbose:
        print(response)


if __name__ == "__main__":
    print("Calling `python -m mlx_lm_amd.generate...` directly is deprecated."
          " Use `python -m mlx_lm_amd generate...` instead.", file=sys.stderr)
    main()
