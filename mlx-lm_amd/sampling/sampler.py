"""Fill the per-row arrays of the sampling kernels from the requests' options."""

import torch

from ..ops import kernels


def _col(values, dtype, device):
    return torch.tensor(values, dtype=dtype, device=device)


def apply_processors(logits, processors, histories):
    """Run each row's logits processors on float32 ``logits [R, V]`` in place.

    ``processors[r]`` is the list for row ``r``, ``histories[r]`` the tokens
    so far (prompt and generated, as the reference passes them,
    mlx_lm/generate.py:400-407).  The built-in kinds (bias, repetition,
    presence and frequency penalties) of all rows go into two kernel
    launches, in the reference's order: biases first, then the penalties;
    any other callable is called on its row.
    """
    from ..sample_utils import FrequencyPenalty, LogitBias, PresencePenalty, RepetitionPenalty

    single = logits.dim() == 1
    if single:
        logits = logits[None]
    R = logits.shape[0]
    dev = logits.device
    bias_off, bias_idx, bias_val = [0], [], []
    rep, rep_ctx, pres, pres_ctx, freq, freq_ctx = ([0.0] * R, [0] * R, [0.0] * R, [0] * R, [0.0] * R, [0] * R)
    hist_off, hist = [0], []
    any_bias = any_pen = False
    custom = []
    for r in range(R):
        span = 0
        for p in processors[r] or ():
            if isinstance(p, LogitBias):
                for t, v in p.bias.items():
                    if not (0 <= t < logits.shape[1]):
                        raise ValueError(f"logit_bias names token {t}, the vocabulary has {logits.shape[1]}")
                    bias_idx.append(t)
                    bias_val.append(v)
                any_bias = True
            elif isinstance(p, RepetitionPenalty):
                rep[r], rep_ctx[r] = float(p.penalty), int(p.context_size)
                span = max(span, p.context_size)
            elif isinstance(p, PresencePenalty):
                pres[r], pres_ctx[r] = float(p.penalty), int(p.context_size)
                span = max(span, p.context_size)
            elif isinstance(p, FrequencyPenalty):
                freq[r], freq_ctx[r] = float(p.penalty), int(p.context_size)
                span = max(span, p.context_size)
            else:
                custom.append((r, p))
        bias_off.append(len(bias_idx))
        if span > 0:
            tail = [int(t) for t in list(histories[r])[-span:]]
            for t in tail:
                if not (0 <= t < logits.shape[1]):
                    raise ValueError(f"a penalty's token history names token {t}, the vocabulary has {logits.shape[1]}")
            hist.extend(tail)
            any_pen = any_pen or bool(tail)
        hist_off.append(len(hist))
    if any_bias:
        kernels.apply_logit_bias(logits, _col(bias_off, torch.int32, dev), _col(bias_idx, torch.int32, dev),
                                 _col(bias_val, torch.float32, dev))
    if any_pen:
        kernels.apply_penalties(
            logits, _col(hist_off, torch.int32, dev), _col(hist, torch.int32, dev),
            _col(rep, torch.float32, dev), _col(rep_ctx, torch.int32, dev),
            _col(pres, torch.float32, dev), _col(pres_ctx, torch.int32, dev),
            _col(freq, torch.float32, dev), _col(freq_ctx, torch.int32, dev))
    for r, p in custom:
        row = p(torch.tensor(list(histories[r]), dtype=torch.int32, device=dev), logits[r : r + 1])
        logits[r : r + 1] = row
    return logits[0] if single else logits


class _ParamRing:
    """Pinned host arrays for the sampling kernel's per-row options, reused in turn.

    One asynchronous copy a call brings all of them to the device, so nothing
    here waits for the GPU; an array is written again only after the copy
    that read it has finished.
    """

    FIELDS = 12  # 32-bit words per row: ten options, and the seed's two halves

    def __init__(self, n=4):
        self.slots = [None] * n
        self.i = 0

    def get(self, rows, device):
        self.i = (self.i + 1) % len(self.slots)
        slot = self.slots[self.i]
        if slot is None or slot[0].numel() < rows * self.FIELDS or slot[1].device != device:
            n = max(rows, 64) * self.FIELDS
            host = torch.empty(n, dtype=torch.int32, pin_memory=True)
            slot = [host, torch.empty(n, dtype=torch.int32, device=device), None]
            self.slots[self.i] = slot
        if slot[2] is not None:
            slot[2].synchronize()
        return slot


class SamplerBuffers:
    """The arrays that sampling calls and the reads of their tokens go through, reused in turn.

    Whoever keeps a call's tokens on the device until its *next* call (a scheduler feeds them
    into the step it launches meanwhile) owns one of these: with at most two calls in flight and
    four arrays in turn, nothing is written again while it is still wanted.  Callers that share
    no owner get arrays of their own for every call.
    """

    def __init__(self, depth=4):
        self.params = _ParamRing(depth)
        self.reads = _ReadRing(depth)


def sample_batch(logits, samplers, seeds, counters, want_logprobs=False, buffers=None):
    """One token for each row of float32 ``logits [R, V]``.

    ``samplers[r]`` is the row's ``Sampler``; ``seeds[r]`` and ``counters[r]``
    key its random numbers, so a row's draw does not depend on the rows beside
    it.  Returns ``(tokens, token_logprobs)`` as device tensors and, with
    ``want_logprobs``, the normalised log-probabilities ``[R, V]`` as a third.
    ``logits - logsumexp(logits)`` then the sampler, as in
    mlx_lm/generate.py:411-412.  Nothing here waits for the GPU.  The returned tokens lie in
    an array of ``buffers`` (a ``SamplerBuffers``) that its fourth call from now writes again;
    without ``buffers`` they lie in arrays made for this call.
    """
    import numpy as np

    R, V = logits.shape
    dev = logits.device
    special = []
    for s in samplers:
        s.check_vocab(V)
        if s.xtc_probability > 0 and s.xtc_special_tokens:
            if special and special != list(s.xtc_special_tokens):
                raise ValueError("rows of one batch must share their xtc_special_tokens")
            special = list(s.xtc_special_tokens)
    slot = (buffers.params if buffers is not None else _ParamRing(1)).get(R, dev)
    host, device_buf = slot[0], slot[1]
    h = host.numpy()
    n = R * _ParamRing.FIELDS
    hf = h[:n].view(np.float32)
    # rows of R words each: 0 temp, 1 top_p, 2 min_p, 3 xtc_prob, 4 xtc_thr (floats);
    # 5 min_keep, 6 top_k, 7 counter (ints); 8..9 the seeds (R 64-bit words); 10 tokens, 11 logprob (out)
    hf[0 * R : 1 * R] = [s.temp for s in samplers]
    hf[1 * R : 2 * R] = [s.top_p for s in samplers]
    hf[2 * R : 3 * R] = [s.min_p for s in samplers]
    hf[3 * R : 4 * R] = [s.xtc_probability for s in samplers]
    hf[4 * R : 5 * R] = [s.xtc_threshold for s in samplers]
    h[5 * R : 6 * R] = [s.min_tokens_to_keep for s in samplers]
    h[6 * R : 7 * R] = [s.top_k for s in samplers]
    h[7 * R : 8 * R] = counters
    h[8 * R : 10 * R].view(np.int64)[:] = [int(x) & 0x7FFFFFFFFFFFFFFF for x in seeds]
    d = device_buf[:n]
    d[: 10 * R].copy_(host[: 10 * R], non_blocking=True)
    ev = slot[2] or torch.cuda.Event()
    ev.record()
    slot[2] = ev
    f = d.view(torch.float32)
    tokens = d[10 * R : 11 * R]
    token_logprob = f[11 * R : 12 * R]
    logprobs = torch.empty((R, V), dtype=torch.float32, device=dev) if want_logprobs else None
    kernels.sample_rows(
        tokens, token_logprob, logits, f[0:R], f[R : 2 * R], f[2 * R : 3 * R], d[5 * R : 6 * R],
        d[6 * R : 7 * R], f[3 * R : 4 * R], f[4 * R : 5 * R], d[8 * R : 10 * R].view(torch.int64),
        d[7 * R : 8 * R], _col(special, torch.int32, dev) if special else None, logprobs)
    # tokens and their log-probabilities lie side by side: one copy brings both to the host
    out = SampledRows(d[10 * R : 12 * R], R)
    if want_logprobs:
        return out.tokens, out.token_logprob, logprobs
    return out.tokens, out.token_logprob


class SampledRows:
    """Tokens and their log-probabilities as one device array (tokens first)."""

    def __init__(self, both, rows):
        self.both, self.rows = both, rows
        self.tokens = both[:rows]
        self.token_logprob = both[rows:].view(torch.float32)


class _ReadRing:
    """Pinned host arrays that sampled tokens are copied into, reused in turn."""

    def __init__(self, n=4):
        self.bufs = [None] * n
        self.i = 0

    def get(self, n_words):
        self.i = (self.i + 1) % len(self.bufs)
        b = self.bufs[self.i]
        if b is None or b.numel() < n_words:
            b = self.bufs[self.i] = torch.empty(max(n_words, 256), dtype=torch.int32, pin_memory=True)
        return b


class PendingRead:
    """Tokens and log-probabilities on their way to the host.

    ``start`` queues the copy behind the sampling kernel and returns at once;
    ``wait`` blocks until that copy (and nothing queued after it) is done, so a
    step launched in between keeps the GPU busy while the host reads.  With
    ``buffers`` (a ``SamplerBuffers``) the host array is one of its four, taken in
    turn; without, one made for this read.
    """

    def __init__(self, tokens, token_logprob, buffers=None):
        R = tokens.numel()
        self.rows = R
        adjacent = (token_logprob.data_ptr() == tokens.data_ptr() + 4 * R and tokens.dtype == torch.int32
                    and tokens.is_contiguous() and token_logprob.is_contiguous())
        self.host = (buffers.reads if buffers is not None else _ReadRing(1)).get(2 * R)
        if adjacent:
            self.host[: 2 * R].copy_(torch.as_strided(tokens, (2 * R,), (1,)), non_blocking=True)
        else:
            self.host[:R].copy_(tokens, non_blocking=True)
            self.host[R : 2 * R].copy_(token_logprob.view(torch.int32), non_blocking=True)
        self.event = torch.cuda.Event()
        self.event.record()

    def wait(self):
        """``(tokens, logprobs)`` as Python lists."""
        import numpy as np

        self.event.synchronize()
        both = self.host.numpy()[: 2 * self.rows]
        return both[: self.rows].tolist(), both[self.rows :].view(np.float32).tolist()


def read_sampled(tokens, token_logprob):
    """``(tokens, logprobs)`` as Python lists, waiting for them (one copy when the two came from one
    ``sample_batch`` call)."""
    return PendingRead(tokens, token_logprob).wait()
