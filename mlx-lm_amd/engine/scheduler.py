"""Continuous batching above the step function.

The reference's ``BatchGenerator`` (mlx_lm/generate.py:1565-1945) keeps a FIFO
of prompts, a prefill batch and a generation batch, and runs them as two
padded model calls per iteration.  Here one ``step`` holds both kinds of work:

1. every decoding request brings its one next token;
2. what is left of ``max_num_batched_tokens`` goes to requests that are still
   reading their prompt, in order of admission, as portions of at most
   ``prefill_step_size`` tokens;
3. waiting requests are admitted, first come first served, while fewer than
   ``max_num_seqs`` run and the pages for their whole prompt are free; those
   pages are taken at admission, so reading a prompt never stalls half-way.

When pages run out for a decoding request, the request admitted last is
pre-empted: its pages are given back and it returns to the *front* of the
waiting queue with everything it has generated kept; when it is admitted again
it reads prompt and generated tokens as one prompt and goes on where it was
(sampling is keyed by the index of the generated token, so the continuation
does not change).  A request that could never fit the pool alone is refused
when it is added.

Decisions (``plan_step``) are pure bookkeeping on the host and can be tested
without a GPU; ``step`` runs a plan through the engine and the sampler.

Where the sampler can work in two phases (``launch`` / ``finish``), steps
overlap the way the reference's loops do with ``mx.async_eval``
(mlx_lm/generate.py:446-451,1449-1456): step t is planned and launched while
the tokens of step t-1 are still on the device (decoding requests get them
fed there), then the host reads the tokens of step t-1, decides who has
finished, and queues the sampling of step t.  ``step`` therefore returns the
outputs of the step before the one it launches.  What cannot be known without
the token -- a stop sequence -- is found a step late: the request has then
taken part in one step too many, whose result is dropped.  What can be known
(``max_tokens``, the model's positions) is: such a request is left out.
"""

import itertools
import time
from collections import deque
from dataclasses import dataclass, field
from typing import Any, Callable, List, Optional, Sequence

from ..cache.manager import OutOfPages, OutOfSlots
from .step import StepEntry

# Every scheduler of the process has a number of its own.  An engine (and its cache manager) may
# serve several schedulers at once -- the reference's ``BatchGenerator`` owns its caches and its
# uid counter (mlx_lm/generate.py:1596-1607,1712-1731), so any number of them are live over one
# model -- and each of them numbers its requests as it likes; the engine knows a request as
# ``(scheduler's number, request_id)``.
_scheduler_numbers = itertools.count()


@dataclass(eq=False)
class Request:
    """One generation request and its progress.

    Two requests are the same only if they are the same object: looking one up
    in the scheduler's lists compares identities, not prompts.
    """

    request_id: Any
    prompt: List[int]
    max_tokens: int
    sampler: Any = None
    logits_processors: Optional[list] = None
    stop_sequences: Sequence[Sequence[int]] = ()
    seed: int = 0
    want_logprobs: bool = False
    # progress
    generated: List[int] = field(default_factory=list)
    num_computed: int = 0  # tokens of prompt+generated whose keys and values are in the cache
    finish_reason: Optional[str] = None
    preemptions: int = 0
    order: int = 0
    # row of the sampling call in flight that holds this request's newest token (not yet in ``generated``)
    inflight_row: Optional[int] = None
    live: bool = False  # the scheduler holds it (waiting or running)
    # the name under which the engine and its cache manager know the request: unique over all
    # schedulers that share the engine (``Scheduler.add`` sets it)
    engine_id: Any = None
    # A kept cache (``prompt_cache.PromptCache``) that the request goes on from and leaves what it
    # computed in: the prompt then holds only the tokens that come on top of the cache's, which
    # are ``offset`` (set when the request is added).
    kept: Any = None
    offset: int = 0
    # Tokens that the kept cache knows but that have not gone through the model yet (the last
    # token of the request before, which ended it before it was fed): this request reads them
    # ahead of its prompt.  Set when the request is added.
    prefix: List[int] = field(default_factory=list)
    # No token is asked for and there is a kept cache: the prompt is read into it and that is all
    # (``generate_step(..., max_tokens=0, prompt_cache=c)`` of the reference reads the whole
    # prompt before it stops, which is how mlx_lm/cache_prompt.py:132-143 fills a cache).
    fill_only: bool = False

    @property
    def tokens(self):
        return self.prompt + self.generated

    @property
    def feed_tokens(self):
        """What goes through the model for this request, in order."""
        return self.prefix + self.prompt + self.generated

    @property
    def num_tokens(self):
        return len(self.prefix) + len(self.prompt) + len(self.generated)

    @property
    def context(self):
        """Tokens of the whole sequence so far, a kept cache's included."""
        return self.offset + len(self.prompt) + len(self.generated)

    @property
    def decoding(self):
        """All but the newest token are computed: the next step brings one token."""
        if self.inflight_row is not None:  # the newest token is still on the device
            return self.num_computed == self.num_tokens
        return self.num_computed == self.num_tokens - 1 and len(self.generated) > 0


@dataclass
class StepOutput:
    """What a step produced for one request (cf. mlx_lm/generate.py:1321-1328)."""

    request_id: Any
    token: int
    logprob: float
    finish_reason: Optional[str] = None
    logprobs: Any = None  # float32 [vocab] device tensor when the request asked for it


@dataclass
class PlannedEntry:
    request: Request
    n_tokens: int
    samples: bool  # the portion ends at the request's newest token: its logits are wanted


@dataclass
class SchedulerStats:
    """Counters and clocks of a scheduler.  A step's wall time counts as prompt time and as
    generation time in proportion to the prompt tokens it read and the tokens it handed out
    (the reference keeps the two apart because it runs them as two model calls,
    mlx_lm/generate.py:1642-1661,1915-1919; here one step holds both)."""

    steps: int = 0
    prompt_tokens: int = 0
    generation_tokens: int = 0
    preemptions: int = 0
    pages_high_water: int = 0
    prompt_time: float = 0.0
    generation_time: float = 0.0

    @property
    def prompt_tps(self):
        return self.prompt_tokens / max(self.prompt_time, 1e-9)

    @property
    def generation_tps(self):
        return self.generation_tokens / max(self.generation_time, 1e-9)


def stops(tokens, stop_sequences):
    """True if ``tokens`` ends with one of the stop sequences.

    The reference matches with a trie over token ids (mlx_lm/generate.py:
    887-956); a suffix comparison finds the same matches.
    """
    for s in stop_sequences:
        n = len(s)
        if n and len(tokens) >= n and list(tokens[-n:]) == list(s):
            return True
    return False


class Scheduler:
    """Admits requests, cuts prompts into portions, decodes, finishes and frees."""

    def __init__(self, engine, sample: Callable, max_num_seqs=32, max_num_batched_tokens=2048,
                 prefill_step_size=2048):
        if max_num_seqs <= 0 or max_num_batched_tokens <= 0 or prefill_step_size <= 0:
            raise ValueError("max_num_seqs, max_num_batched_tokens and prefill_step_size must be positive")
        self.engine = engine
        self.cache = engine.cache
        self.sample = sample
        self.max_positions = engine.decoder.max_positions
        self.max_num_seqs = min(max_num_seqs, self.cache.max_requests)
        self.max_num_batched_tokens = max_num_batched_tokens
        self.prefill_step_size = prefill_step_size
        self.waiting = deque()
        self.running: List[Request] = []
        self.stats = SchedulerStats()
        self._order = 0
        self.number = next(_scheduler_numbers)
        self.pipelined = hasattr(sample, "launch") and hasattr(sample, "finish")
        self._inflight = None  # the sampling call whose tokens the host has not read yet

    # -- requests ----------------------------------------------------------------

    def add(self, request: Request):
        if not request.prompt:
            raise ValueError("a request needs a prompt of at least one token")
        if request.max_tokens < 0:
            raise ValueError("max_tokens must not be negative")
        if request.kept is not None and (request.kept.in_use or getattr(request.kept, "claimed", False)):
            raise ValueError("the request's prompt cache is in use by another request")
        if request.kept is not None and any(g.need.window > 0 for g in self.cache.groups):
            # (pre-emption and removal take a request back to what its cache held; pages that a
            # window has passed are gone, so that state cannot be had again)
            raise ValueError("prompt caches are not offered for a model whose attention has a window")
        if request.kept is not None and getattr(request.kept, "engine", None) not in (None, self.engine):
            raise ValueError("the request's prompt cache holds pages of another engine (another cache "
                             "geometry, dtype or model): it goes on only where it was made")
        request.prefix = list(request.kept.pending) if request.kept is not None else []
        request.offset = request.kept.offset - len(request.prefix) if request.kept is not None else 0
        before = request.offset + len(request.prefix)
        if before + len(request.prompt) > self.max_positions:
            raise ValueError(
                f"the prompt has {len(request.prompt)} tokens"
                + (f" on top of the {before} of its cache" if before else "")
                + f", the model has {self.max_positions} positions"
            )
        most = min(before + len(request.prompt) + request.max_tokens, self.max_positions)
        if self.cache.blocks_for(most) > self.cache.n_pages:
            raise ValueError(
                f"request {request.request_id!r} can reach {most} tokens, the cache holds "
                f"{self.cache.n_pages * self.cache.page_size}"
            )
        if any(r.request_id == request.request_id for r in list(self.waiting) + self.running):
            raise ValueError(f"request id {request.request_id!r} is in use")
        request.order = self._order
        self._order += 1
        request.engine_id = (self.number, request.request_id)
        request.fill_only = request.max_tokens == 0 and request.kept is not None
        if request.max_tokens == 0 and not request.fill_only:
            # nothing to generate and no cache to leave the prompt in: finished as it comes, with
            # no step run and no token sampled (``generate_step`` yields nothing for it,
            # mlx_lm/generate.py:448-461)
            request.finish_reason = "length"
            return request
        request.live = True
        if request.kept is not None:
            request.kept.claimed = True  # (this request's from now on, until it is over)
        self.waiting.append(request)
        return request

    def abort(self, request_id, keep=None):
        """Take a request out, wherever it is (``remove`` of mlx_lm/generate.py:1777-1802).
        ``keep``: an empty kept cache that takes what the request has computed (a request that
        came with a kept cache leaves it there anyway)."""
        if keep is not None and any(g.need.window > 0 for g in self.cache.groups):
            raise ValueError("prompt caches are not offered for a model whose attention has a window")
        for r in list(self.waiting):
            if r.request_id == request_id:
                self.waiting.remove(r)
                r.live = False
                if r.kept is not None:
                    r.kept.claimed = False
                return r
        for r in self.running:
            if r.request_id == request_id:
                if keep is not None and r.kept is None:
                    r.kept, keep.in_use = keep, True
                self._drop(r)
                return r
        raise KeyError(f"request {request_id!r} is not known")

    @property
    def has_work(self):
        return bool(self.waiting or self.running or self._inflight is not None)

    def _drop(self, r):
        r.live = False
        if r in self.running:
            self.running.remove(r)
        elif r in self.waiting:  # pre-empted, and finished by the token that was in flight
            self.waiting.remove(r)
        if r.kept is not None:
            r.kept.claimed = False
        if not self.engine.has_request(r.engine_id):
            return
        if r.kept is None:
            self.engine.end_request(r.engine_id)
        else:
            self._keep(r)

    def _keep(self, r):
        """The request is over and its cache is kept: the cache is to hold exactly the tokens that
        the host knows, the last generated one included (the reference feeds it before it stops,
        mlx_lm/generate.py:444-461).  A token still in flight when the request was taken out is
        forgotten.  The token that ended the request was never fed: the cache keeps it as
        ``pending`` and the next request reads it ahead of its prompt (a step of its own for one
        token would cost every finished request a whole decode step)."""
        eid = r.engine_id
        known = r.context
        have = self.engine.context_len(eid)
        try:
            if have > known:
                r.kept.rewind(self.engine, eid, known)
                have = self.engine.context_len(eid)
        finally:
            r.kept.checkin(self.engine, eid)
        fed = have - r.offset  # of prefix + prompt + generated
        if r.finish_reason is not None:
            r.kept.pending = r.feed_tokens[fed:]
        else:  # taken out half-way: what was computed, and of the cache's own pending tokens those not yet read
            r.kept.pending = r.prefix[fed:]

    def close(self):
        """Take every request out and give back what they hold in the engine."""
        self._inflight = None
        for r in list(self.waiting) + list(self.running):
            self._drop(r)

    def _ends_with_token_in_flight(self, r):
        """The token in flight is the request's last, whatever it is."""
        return r.inflight_row is not None and (
            len(r.generated) + 1 >= r.max_tokens or r.context + 1 >= self.max_positions)

    def _preempt(self, r):
        if r.kept is not None and self.engine.has_request(r.engine_id):
            # back to what the kept cache held when the request came: only its own tokens are read again
            r.kept.rewind(self.engine, r.engine_id)
            r.kept.checkin(self.engine, r.engine_id)
            r.kept.pending = list(r.prefix)
        self._drop(r)
        r.num_computed = 0
        r.preemptions += 1
        self.stats.preemptions += 1
        r.live = True
        if r.kept is not None:
            r.kept.claimed = True
        self.waiting.appendleft(r)

    # -- decisions ---------------------------------------------------------------

    def _pages_for(self, r, n_new):
        if self.engine.has_request(r.engine_id):
            return self.cache.pages_needed(r.engine_id, n_new)
        return self.cache.blocks_for(n_new)

    def plan_step(self):
        """Decide what the next step runs; may pre-empt.  Returns ``[PlannedEntry]``."""
        free = self.cache.free_pages()
        budget = self.max_num_batched_tokens
        plan = []

        # 1. one token for every decoding request; pre-empt from the newest if pages run short
        decoding = [r for r in self.running if r.decoding and not self._ends_with_token_in_flight(r)]
        decoding.sort(key=lambda r: r.order)
        while decoding:
            need = sum(self._pages_for(r, 1) for r in decoding)
            if need <= free and len(decoding) <= budget:
                break
            victim = max(self.running, key=lambda r: r.order)
            if victim in decoding:
                decoding.remove(victim)
            self._preempt(victim)
            free = self.cache.free_pages()
        for r in decoding:
            free -= self._pages_for(r, 1)
            budget -= 1
            plan.append(PlannedEntry(r, 1, True))

        # 2. requests still reading their prompt, in order of admission
        for r in sorted((r for r in self.running if not r.decoding), key=lambda r: r.order):
            if budget <= 0:
                break
            left = r.num_tokens - r.num_computed
            n = min(left, budget, self.prefill_step_size)
            while n > 0 and self._pages_for(r, n) > free:
                n = self._fit(r, n, free)
            if n <= 0:
                continue
            free -= self._pages_for(r, n)
            budget -= n
            plan.append(PlannedEntry(r, n, n == left and not r.fill_only))

        # 3. admit waiting requests while their whole prompt fits
        while self.waiting and len(self.running) < self.max_num_seqs and budget > 0:
            r = self.waiting[0]
            if r.inflight_row is not None:
                break  # pre-empted with a token in flight: it is read as a prompt once that token is known
            # (a kept cache brings the pages of its tokens with it)
            n_new = min(r.num_tokens + (0 if r.fill_only else 1), self.max_positions - r.offset)
            whole = self.cache.blocks_for(r.offset + n_new) - self.cache.blocks_for(r.offset)
            if r.kept is not None and getattr(r.kept, "needs_pages", False):
                whole += self.cache.blocks_for(r.offset)  # (read from a file: its tokens have no pages yet)
            if whole > free:
                break
            # The request leaves the queue only once the engine has it and its pages: whatever
            # goes wrong before (another scheduler on the same engine holds the last slot) leaves
            # it waiting, first in line.  The whole prompt's pages are taken now, so a request that
            # was admitted can always finish reading its prompt.
            try:
                if r.kept is not None:
                    r.kept.checkout(self.engine, r.engine_id)
                else:
                    self.engine.add_request(r.engine_id)
            except (OutOfSlots, OutOfPages):
                break
            try:
                self.cache.reserve(r.engine_id, n_new)
            except BaseException as e:
                if r.kept is not None:
                    r.kept.checkin(self.engine, r.engine_id)
                    r.kept.pending = list(r.prefix)
                else:
                    self.engine.end_request(r.engine_id)
                if isinstance(e, OutOfPages):
                    break
                raise
            self.waiting.popleft()
            self.running.append(r)
            n = min(r.num_tokens, budget, self.prefill_step_size)
            free -= whole
            budget -= n
            plan.append(PlannedEntry(r, n, n == r.num_tokens and not r.fill_only))
        return plan

    def _fit(self, r, n, free):
        """The longest portion of at most ``n`` tokens whose pages are free."""
        ps = self.cache.page_size
        if self.engine.has_request(r.engine_id):
            rc = self.cache.requests[r.engine_id]
            room = self.cache.blocks_for(rc.reserved) * ps - rc.length
        else:
            room = 0
        return min(n - 1, room + free * ps)

    # -- running a plan ------------------------------------------------------------

    def step(self):
        """Plan, run and sample one step; returns the ``StepOutput`` of every sampled token
        (of this step, or of the step before where steps overlap)."""
        tic = time.perf_counter()
        prompt_before = self.stats.prompt_tokens
        outputs = self._step()
        elapsed = time.perf_counter() - tic
        read, made = self.stats.prompt_tokens - prompt_before, len(outputs)
        if read + made:
            self.stats.prompt_time += elapsed * read / (read + made)
            self.stats.generation_time += elapsed * made / (read + made)
        return outputs

    def _step(self):
        if not self.pipelined:
            return self._step_in_turn()
        prev, self._inflight = self._inflight, None
        outputs = []
        if prev is not None and not prev.feedable:
            outputs = self._finish(prev)  # tokens made on the host: nothing to overlap
            prev = None
        plan = self.plan_step()
        logits = None
        if plan:
            logits = self._run(plan, prev)
        elif prev is None and self.has_work and not self.running:
            raise RuntimeError(self._stuck())
        if prev is not None:
            outputs = self._finish(prev)  # the GPU is busy with this step meanwhile
        sampled = [p.request for p in plan if p.samples]
        if sampled:
            job = self.sample.launch(logits, sampled)
            for i, r in enumerate(sampled):
                r.inflight_row = i
            self._inflight = job
        return outputs

    def _stuck(self):
        """Why nothing can run: requests wait, none runs here, and the first in line finds no room
        (``add`` refused what could never fit, so others on the same engine hold the room)."""
        others = [rid for rid in self.cache.requests
                  if not (isinstance(rid, tuple) and len(rid) == 2 and rid[0] == self.number)]
        kept = sum(len(pages) for k in getattr(self.cache, "kept", ()) for pages in k.blocks)
        return (f"requests are waiting but none can be admitted: {self.cache.free_pages()} of "
                f"{self.cache.n_pages} pages are free, {len(others)} requests of other generators "
                f"on this engine hold pages or slots and kept prompt caches hold {kept} pages; "
                f"finish, close or free those first")

    def _run(self, plan, prev=None):
        """Launch the planned step; decoding requests whose token is in flight get it fed on the device."""
        entries = []
        for p in plan:
            r = p.request
            if r.inflight_row is not None:
                entries.append(StepEntry(r.engine_id, [0], [0] if p.samples else [], fed_row=r.inflight_row))
            else:
                toks = r.feed_tokens[r.num_computed : r.num_computed + p.n_tokens]
                entries.append(StepEntry(r.engine_id, toks, [p.n_tokens - 1] if p.samples else []))
        if prev is not None and any(e.fed_row >= 0 for e in entries):
            logits = self.engine.step(entries, fed=prev.tokens)
        else:
            logits = self.engine.step(entries)
        for p in plan:
            r = p.request
            if not r.generated and r.inflight_row is None:
                self.stats.prompt_tokens += p.n_tokens
            r.num_computed += p.n_tokens
            if r.fill_only and r.num_computed >= r.num_tokens:  # the prompt is in its cache: done
                r.finish_reason = "length"
                self._drop(r)
        self.stats.steps += 1
        self.stats.pages_high_water = max(
            self.stats.pages_high_water, max((g.pool.high_water for g in self.cache.groups), default=0)
        )
        return logits

    def _finish(self, job):
        """Read a sampling call's tokens and give them to their requests."""
        results = self.sample.finish(job)
        outputs = []
        for r, (token, logprob, logprobs) in zip(job.requests, results):
            r.inflight_row = None
            if r.finish_reason is not None or not r.live:
                continue  # finished a step ago (this token is one too many), or taken out meanwhile
            outputs.append(self._take(r, token, logprob, logprobs))
        return outputs

    def _take(self, r, token, logprob, logprobs):
        r.generated.append(int(token))
        self.stats.generation_tokens += 1
        # "length" at max_tokens or when the model's positions are used up;
        # "stop" is checked second and wins (mlx_lm/generate.py:1501-1514)
        reason = None
        if len(r.generated) >= r.max_tokens or r.context >= self.max_positions:
            reason = "length"
        if stops(r.generated, r.stop_sequences):
            reason = "stop"
        r.finish_reason = reason
        if reason is not None:
            self._drop(r)
        return StepOutput(r.request_id, int(token), float(logprob), reason, logprobs)

    def _step_in_turn(self):
        """One step and its sampling, the host waiting for the tokens before it goes on."""
        plan = self.plan_step()
        if not plan:
            if self.has_work and not self.running:
                raise RuntimeError(self._stuck())
            return []
        logits = self._run(plan)
        sampled = [p.request for p in plan if p.samples]
        if not sampled:
            return []
        results = self.sample(logits, sampled)
        return [self._take(r, token, logprob, logprobs)
                for r, (token, logprob, logprobs) in zip(sampled, results)]
