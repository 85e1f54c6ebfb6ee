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
            tail = list(histories[r])[-span:]
            hist.extend(int(t) for t in tail)
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


def sample_batch(logits, samplers, seeds, counters, want_logprobs=False):
    """One token for each row of float32 ``logits [R, V]``.

    ``samplers[r]`` is the row's ``Sampler``; ``seeds[r]`` and ``counters[r]``
    key its random numbers, so a row's draw does not depend on the rows beside
    it.  Returns ``(tokens, token_logprobs)`` as device tensors and, with
    ``want_logprobs``, the normalised log-probabilities ``[R, V]`` as a third.
    ``logits - logsumexp(logits)`` then the sampler, as in
    mlx_lm/generate.py:411-412.
    """
    R, V = logits.shape
    dev = logits.device
    special = []
    for s in samplers:
        s.check_vocab(V)
        if s.xtc_probability > 0 and s.xtc_special_tokens:
            if special and special != list(s.xtc_special_tokens):
                raise ValueError("rows of one batch must share their xtc_special_tokens")
            special = list(s.xtc_special_tokens)
    tokens = torch.empty(R, dtype=torch.int32, device=dev)
    token_logprob = torch.empty(R, dtype=torch.float32, device=dev)
    logprobs = torch.empty((R, V), dtype=torch.float32, device=dev) if want_logprobs else None
    f32 = lambda name: _col([float(getattr(s, name)) for s in samplers], torch.float32, dev)
    i32 = lambda name: _col([int(getattr(s, name)) for s in samplers], torch.int32, dev)
    kernels.sample_rows(
        tokens, token_logprob, logits, f32("temp"), f32("top_p"), f32("min_p"),
        i32("min_tokens_to_keep"), i32("top_k"), f32("xtc_probability"), f32("xtc_threshold"),
        _col([int(x) & 0x7FFFFFFFFFFFFFFF for x in seeds], torch.int64, dev),
        _col([int(c) for c in counters], torch.int32, dev),
        _col(special, torch.int32, dev) if special else None, logprobs)
    if want_logprobs:
        return tokens, token_logprob, logprobs
    return tokens, token_logprob
