"""Generation: ``generate_step``, ``stream_generate``, ``generate``,
``BatchGenerator``, ``batch_generate`` and the ``generate`` command line,
with the names and meanings of mlx_lm/generate.py.

All of them run on the continuous-batching scheduler and the step function of
``mlx_lm_amd.engine``; a single request is a batch of one.
"""

import argparse
import contextlib
import dataclasses
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
    "max_kv_size": None, "kv_bits": None, "input_embeddings": None,
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


class _OneRequest:
    """One prompt on a scheduler of its own: iterating yields the ``StepOutput`` of every token.

    The prompt is read in portions of ``prefill_step_size`` (under ``max_num_batched_tokens``
    a step); then one token per step.  ``stop_tokens`` end the request with reason ``"stop"``,
    ``max_tokens`` or the model's positions with ``"length"``; its pages go back at once.
    ``page_size``/``num_pages`` choose the cache that the model's engine is made with; ``engine``
    names an engine instead (by default the one whose pool ``prompt_cache`` lies in, if it holds tokens).
    ``prompt_cache`` (a ``PromptCache``): the prompt comes on top of the tokens that the cache
    holds, and when the request ends the cache holds the prompt and all generated tokens as well.
    """

    def __init__(self, model, prompt, max_tokens, sampler=None, logits_processors=None,
                 prefill_step_size=2048, prompt_progress_callback=None, seed=None, stop_tokens=(),
                 want_logprobs=True, page_size=16, num_pages=None, max_num_seqs=1,
                 max_num_batched_tokens=None, prompt_cache=None, engine=None):
        self.prompt = [int(t) for t in (prompt.tolist() if hasattr(prompt, "tolist") else prompt)]
        if len(self.prompt) == 0:
            raise ValueError("Either input_embeddings or prompt (or both) must be provided.")
        if engine is None and prompt_cache is not None:
            engine = prompt_cache.engine  # a cache that holds tokens holds them in one engine's pool
        self.engine = engine or engine_for(
            model, page_size=page_size, max_cache_tokens=None if num_pages is None else num_pages * page_size)
        self.scheduler = Scheduler(self.engine, make_sample_fn(), max_num_seqs=max(1, max_num_seqs),
                                   max_num_batched_tokens=max_num_batched_tokens or prefill_step_size,
                                   prefill_step_size=prefill_step_size)
        _uid[0] += 1
        self.request_id = ("generate_step", _uid[0])
        if seed is None:
            seed = getattr(sampler, "seed", None)
        if seed is None:
            seed = sample_utils.default_seed()
        self.request = Request(self.request_id, self.prompt, max_tokens, sampler=sampler,
                               logits_processors=logits_processors, seed=seed, want_logprobs=want_logprobs,
                               stop_sequences=[[int(t)] for t in stop_tokens], kept=prompt_cache)
        self.progress = prompt_progress_callback
        self.scheduler.add(self.request)

    @property
    def stats(self):
        return self.scheduler.stats

    def __iter__(self):
        sched, req = self.scheduler, self.request
        try:
            while sched.has_work:
                outs = sched.step()
                if self.progress is not None and not req.generated:
                    read = max(0, req.num_computed - len(req.prefix))  # (of the prompt itself)
                    self.progress(min(read, len(self.prompt)), len(self.prompt))
                yield from outs
        finally:
            sched.close()  # (a generator dropped half-way gives its pages back here)


def generate_step(prompt, model, *, max_tokens=256, sampler=None, logits_processors=None,
                  prefill_step_size=2048, prompt_progress_callback=None, seed=None, prompt_cache=None,
                  **kwargs):
    """Yield ``(token, logprobs)`` for one prompt (mlx_lm/generate.py:298-461).

    ``prompt_cache`` (``make_prompt_cache(model)``): what earlier calls computed; the prompt is
    read on top of it and the cache is updated in place (mlx_lm/generate.py:306,329-331), so a
    later call goes on from prompt and generated tokens with only its own tokens to read.

    The prompt is read in portions of ``prefill_step_size``; then one token
    per step.  ``logprobs`` is a float32 device tensor ``[vocab]``.  Exactly
    ``max_tokens`` tokens are yielded unless the model's positions run out.
    Beyond the reference's options: ``seed`` keys the draws; ``page_size``,
    ``num_pages``, ``max_num_seqs`` and ``max_num_batched_tokens`` shape the
    cache and the scheduler; ``engine`` names the engine to run on.
    """
    _refuse_unsupported(kwargs)
    geometry = {k: kwargs.pop(k) for k in _ENGINE_OPTIONS if k in kwargs}
    if kwargs:
        raise TypeError(f"unknown options: {sorted(kwargs)}")
    run = _OneRequest(model, prompt, max_tokens, sampler=sampler, logits_processors=logits_processors,
                      prefill_step_size=prefill_step_size, prompt_progress_callback=prompt_progress_callback,
                      seed=seed, prompt_cache=prompt_cache, **geometry)
    for out in run:
        yield out.token, out.logprobs


_ENGINE_OPTIONS = ("page_size", "num_pages", "max_num_seqs", "max_num_batched_tokens", "engine")


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
    after ``max_tokens``; the last response carries ``finish_reason``.  The end
    tokens are the request's stop tokens, so the scheduler ends it (and gives
    its pages back) with the token that ends it; rates come from the
    scheduler's clocks: the prompt's up to the first token, the generation's
    from there.
    """
    if draft_model is not None:
        raise ValueError("speculative decoding is not supported")
    tokenizer = tokenizer if tokenizer is not None else IdTokenizer()
    if isinstance(prompt, str):
        bos = tokenizer.bos_token
        prompt = tokenizer.encode(prompt, add_special_tokens=bos is None or not prompt.startswith(bos))
    _refuse_unsupported(kwargs)
    run = _OneRequest(model, prompt, max_tokens, stop_tokens=sorted(tokenizer.eos_token_ids), **kwargs)
    detokenizer = tokenizer.detokenizer
    started = first_token_at = time.perf_counter()
    made = 0

    def response(out, reason):
        now = time.perf_counter()
        return GenerationResponse(
            text=detokenizer.last_segment, token=out.token, logprobs=out.logprobs, from_draft=False,
            prompt_tokens=len(run.prompt), prompt_tps=len(run.prompt) / max(first_token_at - started, 1e-9),
            generation_tokens=made, generation_tps=made / max(now - first_token_at, 1e-9),
            peak_memory=_peak_memory_gb(), finish_reason=reason)

    for out in run:
        if made == 0:
            first_token_at = time.perf_counter()
        made += 1
        if out.finish_reason != "stop":  # the token that stops the request is not part of the text
            detokenizer.add_token(out.token)
        if out.finish_reason is not None:
            detokenizer.finalize()
        yield response(out, out.finish_reason)


def generate(model, tokenizer, prompt, verbose=False, **kwargs):
    """The whole response as text (mlx_lm/generate.py:747-790).

    Without a tokenizer the text is the generated token ids in decimal.
    """
    rule = "=" * 10
    pieces, last = [], None
    if verbose:
        print(rule)
    for last in stream_generate(model, tokenizer, prompt, **kwargs):
        pieces.append(last.text)
        if verbose:
            print(last.text, end="", flush=True)
    text = "".join(pieces)
    if not verbose:
        return text
    print()
    print(rule)
    if not text:
        print("No text generated for this prompt")
        return
    print(f"Prompt: {last.prompt_tokens} tokens, {last.prompt_tps:.3f} tokens-per-sec")
    print(f"Generation: {last.generation_tokens} tokens, {last.generation_tps:.3f} tokens-per-sec")
    print(f"Peak memory: {last.peak_memory:.3f} GB")
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
                 want_logprobs=True, engine=None, return_prompt_caches=False):
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
        # every finished request's response carries what it computed as a ``PromptCache``
        self.return_prompt_caches = return_prompt_caches

    def close(self):
        """Drop every request; their pages and slots go back to the engine, which other
        generators over the same model share."""
        live, self._requests = list(self._requests.values()), {}
        self.scheduler.close()
        for r in live:
            if r.kept is not None:
                r.kept.free()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @contextlib.contextmanager
    def stats(self, stats=None):
        """Counts and rates of what runs inside the ``with`` (mlx_lm/generate.py:1642-1661), from
        the scheduler's counters and clocks."""
        stats = stats or BatchStats()
        before = dataclasses.replace(self.scheduler.stats)
        try:
            yield stats
        finally:
            now = self.scheduler.stats
            stats.prompt_tokens += now.prompt_tokens - before.prompt_tokens
            stats.prompt_time += now.prompt_time - before.prompt_time
            stats.prompt_tps = stats.prompt_tokens / max(stats.prompt_time, 1e-9)
            stats.generation_tokens += now.generation_tokens - before.generation_tokens
            stats.generation_time += now.generation_time - before.generation_time
            stats.generation_tps = stats.generation_tokens / max(stats.generation_time, 1e-9)
            stats.peak_memory = max(stats.peak_memory, _peak_memory_gb())

    def insert(self, prompts, max_tokens=None, caches=None, all_tokens=None, samplers=None,
               logits_processors=None, stop_matchers=None, seeds=None):
        """Queue prompts; per-request lists override the generator's defaults.

        ``stop_matchers[i]`` is a list of token-id sequences that stop request
        ``i``.  ``seeds[i]`` keys its random draws (default: the generator's
        seed plus the uid).  ``caches[i]``: a ``PromptCache`` that request ``i`` goes on from: its
        prompt comes on top of the cache's tokens.  As in the reference, which merges the given
        caches into its batch (mlx_lm/generate.py:1107-1120), the cache given stays as it is:
        the request works on a copy (pages of its own), which its last response carries.
        """
        from .prompt_cache import PromptCache

        for c in caches or ():
            if c is not None and c.engine not in (None, self.engine):
                raise ValueError("a prompt cache in 'caches' holds pages of another engine than this "
                                 "generator's: it goes on only where it was made")
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
                want_logprobs=self.want_logprobs,
                kept=(caches[i].copy() if caches and caches[i] is not None
                      else PromptCache(self.model) if self.return_prompt_caches else None))
            self.scheduler.add(req)
            if req.finish_reason is None:  # (a request for no tokens at all is over already)
                self._requests[uid] = req
            uids.append(uid)
        return uids

    def remove(self, uids, return_prompt_caches=False):
        """Drop requests; with ``return_prompt_caches`` a dict from uid to the ``PromptCache`` of
        what the request had computed (mlx_lm/generate.py:1777-1802)."""
        from .prompt_cache import PromptCache

        caches = {}
        for uid in uids:
            if uid in self._requests:
                r = self._requests.pop(uid)
                keep = PromptCache(self.model) if return_prompt_caches and r.kept is None else None
                try:
                    self.scheduler.abort(uid, keep=keep)
                except KeyError:
                    pass
                if return_prompt_caches and r.kept is not None:
                    caches[uid] = r.kept
                elif r.kept is not None:
                    r.kept.free()  # the request's own copy: nobody goes on from it
        return caches if return_prompt_caches else None

    def _next(self):
        before = {uid: r.num_computed for uid, r in self._requests.items() if not r.generated}
        outs = self.scheduler.step()
        prompt_responses = []
        for uid, done in before.items():
            r = self._requests[uid]
            if r.num_computed != done:
                n, read = len(r.prompt), max(0, r.num_computed - len(r.prefix))
                prompt_responses.append(self.PromptResponse(uid, (min(read, n), n), read >= n))
        responses = []
        for o in outs:
            r = self._requests[o.request_id]
            responses.append(self.Response(o.request_id, o.token, o.logprobs, o.finish_reason,
                                           r.kept if o.finish_reason else None,
                                           r.tokens if o.finish_reason else None, o.logprob))
            if o.finish_reason is not None:
                del self._requests[o.request_id]
        # a request for no tokens on top of a cache is over once its prompt is read: its one
        # response carries no token, only the cache
        for uid, r in list(self._requests.items()):
            if r.fill_only and r.finish_reason is not None:
                responses.append(self.Response(uid, None, None, r.finish_reason, r.kept, r.tokens))
                del self._requests[uid]
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
    """Run a list of prompts to completion (mlx_lm/generate.py:1971-2060).

    The tokenizer's end tokens stop a request; the token that stops it is not part of its
    result.  ``kwargs`` go to ``BatchGenerator``.
    """
    tokenizer = tokenizer if tokenizer is not None else IdTokenizer()
    gen = BatchGenerator(model, stop_tokens=[[t] for t in tokenizer.eos_token_ids],
                         want_logprobs=False, return_prompt_caches=return_prompt_caches, **kwargs)
    limits = [max_tokens] * len(prompts) if isinstance(max_tokens, int) else list(max_tokens)
    total, finished = len(prompts), 0

    def progress(end="\r"):
        if verbose:
            print(f"[batch_generate] Finished processing {finished}/{total}" + (" ..." if end == "\r" else ""),
                  end=end)

    progress()
    uids = gen.insert(prompts, limits, caches=prompt_caches)
    kept = {uid: ([], []) for uid in uids}  # tokens and their log-probabilities
    caches = {}
    with gen.stats() as stats:
        while True:
            responses = gen.next_generated()
            if not responses:
                break
            for r in responses:
                if r.finish_reason != "stop" and r.token is not None:
                    kept[r.uid][0].append(r.token)
                    kept[r.uid][1].append(r.token_logprob)
                if r.finish_reason is not None:
                    finished += 1
                    caches[r.uid] = r.prompt_cache
                    progress()
    gen.close()
    if not return_prompt_caches:
        for c in caches.values():
            if c is not None:
                c.free()
    progress(end="\n")
    if verbose:
        print(f"[batch_generate] Prompt: {stats.prompt_tokens} tokens, {stats.prompt_tps:.3f} tokens-per-sec")
        print(f"[batch_generate] Generation: {stats.generation_tokens} tokens, "
              f"{stats.generation_tps:.3f} tokens-per-sec")
        print(f"[batch_generate] Peak memory: {stats.peak_memory:.3f} GB")
    return BatchResponse([tokenizer.decode(kept[uid][0]) for uid in uids], stats,
                         [caches.get(uid) for uid in uids] if return_prompt_caches else None,
                         [kept[uid][0] for uid in uids] if return_token_ids else None,
                         [kept[uid][1] for uid in uids] if return_logprobs else None)


# ---------------------------------------------------------------------------
# command line


def str2bool(string):
    return string.lower() not in ["false", "f"]


# The options of ``mlx_lm.generate`` that this engine has (mlx_lm/generate.py:54-213), with the
# reference's names, defaults and meanings, then the engine's own.  (flags, type, default, help, more)
_OPTIONS = [
    (("--model",), str, None, "A local model folder (config.json, model.safetensors); not needed with --random-weights.", {}),
    (("--extra-eos-token",), str, (), "More tokens that end the generation.", {"nargs": "+"}),
    (("--system-prompt",), None, None, "A system message for the tokenizer's chat template.", {}),
    (("--prompt", "-p"), None, DEFAULT_PROMPT, "The message to answer ('-' reads it from standard input).", {}),
    (("--prompt-ids",), str, None, "The prompt as token ids, separated by commas or spaces "
                                   "(for model folders without a tokenizer).", {}),
    (("--prefill-response",), None, None, "A start of the answer, which the model goes on from.", {}),
    (("--max-tokens", "-m"), int, DEFAULT_MAX_TOKENS, "The most tokens to generate.", {}),
    (("--temp",), float, DEFAULT_TEMP, "Sampling temperature (0: the most likely token).", {}),
    (("--top-p",), float, DEFAULT_TOP_P, "Sample from the most likely tokens that hold this much probability.", {}),
    (("--min-p",), float, DEFAULT_MIN_P, "Drop tokens less likely than this fraction of the most likely one's probability.", {}),
    (("--top-k",), int, DEFAULT_TOP_K, "Sample from the k most likely tokens (0: all).", {}),
    (("--xtc-probability",), float, DEFAULT_XTC_PROBABILITY, "How often XTC sampling drops the top choices.", {}),
    (("--xtc-threshold",), float, 0.1, "XTC drops all but the least likely of the tokens above this probability.", {}),
    (("--min-tokens-to-keep",), int, DEFAULT_MIN_TOKENS_TO_KEEP, "What min-p leaves at least.", {}),
    (("--seed",), int, DEFAULT_SEED, "Seed of the random draws.", {}),
    (("--ignore-chat-template",), None, False, "Give the model the prompt as it is.", {"action": "store_true"}),
    (("--chat-template-config",), None, None, "More variables for the chat template, as a JSON object.", {}),
    (("--prompt-cache-file",), str, None, "A file containing saved KV caches to avoid recomputing them "
                                          "(written by the cache_prompt command): the prompt goes on from it.", {}),
    (("--verbose",), str2bool, True, "'True'/'T': stream the text, then print token counts, rates and peak "
                                     "memory; 'False'/'F': print the text only.", {}),
    # this engine's own
    (("--dtype",), None, "bfloat16", "Precision of the weights and the arithmetic.", {"choices": ["bfloat16", "float32"]}),
    (("--prefill-step-size",), int, 2048, "The most tokens of the prompt that one step reads.", {}),
    (("--block-size",), int, 16, "Tokens per page of the key/value cache (a multiple of 16).", {}),
    (("--num-pages",), int, None, "Pages of the cache pool (default: room for 64 full contexts, within memory).", {}),
    (("--max-num-seqs",), int, 1, "The most requests that run at a time.", {}),
    (("--max-num-batched-tokens",), int, None, "The most tokens of one step (default: --prefill-step-size).", {}),
    (("--random-weights",), int, None, "Draw the weights with this seed for the configuration given by --config "
                                      "(or by --model's config.json) instead of reading them.", {"metavar": "SEED"}),
    (("--config",), str, None, "A config.json for --random-weights.", {}),
]


def setup_arg_parser():
    parser = argparse.ArgumentParser(description="LLM inference script")
    for flags, kind, default, text, more in _OPTIONS:
        options = dict(default=default, help=text, **more)
        if kind is not None:
            options["type"] = kind
        parser.add_argument(*flags, **options)
    return parser


def chat_prompt(tokenizer, prompt, args, using_cache=False):
    """The prompt inside the tokenizer's chat template, as token ids (mlx_lm/generate.py:2115-2152).

    A tokenizer without a template, or ``--ignore-chat-template``, leaves the text as it is.
    ``using_cache``: what comes before the user's text in the template lies in a saved cache
    already, so the prompt is the template's text from the last message's text on (2139-2149).
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
    if using_cache:
        text = tokenizer.apply_chat_template(messages, tokenize=False, continue_final_message=has_prefill,
                                             add_generation_prompt=not has_prefill, **template_kwargs)
        marked = [dict(m) for m in messages]
        marked[-1]["content"] = "<query>"
        probe = tokenizer.apply_chat_template(marked, tokenize=False, continue_final_message=has_prefill,
                                              add_generation_prompt=not has_prefill)
        return tokenizer.encode(text[probe.index("<query>"):], add_special_tokens=False)
    return tokenizer.apply_chat_template(messages, tokenize=True, continue_final_message=has_prefill,
                                         add_generation_prompt=not has_prefill, **template_kwargs)


def _model_of(args):
    """The model and tokenizer that the command line names: a folder's, or random weights for a configuration."""
    from .utils import load, load_config, model_from_tensors

    if args.random_weights is None:
        if args.model is None:
            raise SystemExit("give --model DIR (or --random-weights SEED with --config FILE)")
        return load(args.model, dtype=args.dtype)
    if args.config is not None:
        with open(args.config) as fh:
            config = json.load(fh)
    elif args.model is not None:
        config = load_config(args.model)
    else:
        raise SystemExit("--random-weights needs --config FILE or --model DIR for the configuration")
    from .config import get_model_classes

    model_cls, args_cls = get_model_classes(config)
    tensors = model_cls.random_weights(args_cls.from_dict(config), args.random_weights, "b")
    return model_from_tensors(config, tensors, dtype=args.dtype), None


def main(argv=None):
    args = setup_arg_parser().parse_args(argv)
    if args.seed is not None:
        sample_utils.seed(args.seed)
    prompt_cache = None
    if args.prompt_cache_file is not None:
        # the cache, and the model it was made with unless another is named (mlx_lm/generate.py:2070-2096)
        from .prompt_cache import load_prompt_cache

        prompt_cache, metadata = load_prompt_cache(args.prompt_cache_file, return_metadata=True)
        if args.model is None and args.random_weights is None and metadata.get("model"):
            args.model = metadata["model"]
    model, tokenizer = _model_of(args)
    tokenizer = tokenizer if tokenizer is not None else IdTokenizer()
    for token in args.extra_eos_token:
        tokenizer.add_eos_token(token)
    if args.prompt_ids is not None:
        prompt = [int(t) for t in args.prompt_ids.replace(",", " ").split()]
    else:
        text = args.prompt.replace("\\n", "\n").replace("\\t", "\t")
        prompt = chat_prompt(tokenizer, sys.stdin.read() if text == "-" else text, args,
                             using_cache=prompt_cache is not None)
    never_dropped = []  # by XTC: the line break and the end tokens (mlx_lm/generate.py:2168)
    if args.xtc_probability > 0:
        never_dropped = list(tokenizer.encode("\n", add_special_tokens=False)) + sorted(tokenizer.eos_token_ids)
    sampler = make_sampler(args.temp, args.top_p, args.min_p, args.min_tokens_to_keep, top_k=args.top_k,
                           xtc_probability=args.xtc_probability, xtc_threshold=args.xtc_threshold,
                           xtc_special_tokens=never_dropped)
    text = generate(model, tokenizer, prompt, max_tokens=args.max_tokens, verbose=args.verbose, sampler=sampler,
                    prompt_cache=prompt_cache, prefill_step_size=args.prefill_step_size, page_size=args.block_size, num_pages=args.num_pages,
                    max_num_seqs=args.max_num_seqs, max_num_batched_tokens=args.max_num_batched_tokens)
    if not args.verbose:
        print(text)


if __name__ == "__main__":
    print("Calling `python -m mlx_lm_amd.generate...` directly is deprecated."
          " Use `python -m mlx_lm_amd generate...` instead.", file=sys.stderr)
    main()
