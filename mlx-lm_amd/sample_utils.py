"""Samplers and logits processors, with the reference's names and meanings.

``make_sampler`` and ``make_logits_processors`` take the options of
mlx_lm/sample_utils.py:10-126.  What they return are small objects that hold
the options: the scheduler reads them to fill the per-row arrays of one
batched sampling kernel, and they can also be called directly on device
tensors, as the reference's closures are.
"""

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch


@dataclass
class Sampler:
    """Sampling options of one request (mlx_lm/sample_utils.py:10-69).

    ``temp == 0`` is argmax.  Otherwise the filters apply in the reference's
    order, top_p, min_p, xtc, top_k, and a token is drawn from
    ``softmax(filtered / temp)``.  Calling the object on log-probabilities
    ``[B, V]`` (a float32 device tensor) returns int32 tokens ``[B]``.
    """

    temp: float = 0.0
    top_p: float = 0.0
    min_p: float = 0.0
    min_tokens_to_keep: int = 1
    top_k: int = 0
    xtc_probability: float = 0.0
    xtc_threshold: float = 0.1
    xtc_special_tokens: List[int] = field(default_factory=list)
    seed: Optional[int] = None
    _calls: int = 0

    def __post_init__(self):
        if self.temp < 0:
            raise ValueError(f"`temp` must not be negative, but is {self.temp}")
        if not (0 <= self.min_p <= 1.0):
            raise ValueError(f"`min_p` has to be a float in the [0, 1] interval, but is {self.min_p}")
        if not isinstance(self.min_tokens_to_keep, int) or self.min_tokens_to_keep < 1:
            raise ValueError(
                f"`min_tokens_to_keep` has to be a positive integer, but is {self.min_tokens_to_keep}"
            )
        if not (0 <= self.xtc_threshold <= 0.5):
            raise ValueError(
                f"`threshold` has to be a float in the [0, 0.5] interval, but is {self.xtc_threshold}"
            )
        if not (0 <= self.xtc_probability <= 1.0):
            raise ValueError(
                f"`probability` has to be a float in the [0, 1] interval, but is {self.xtc_probability}"
            )
        if not isinstance(self.top_k, int) or self.top_k < 0:
            raise ValueError(f"`top_k` has to be a non-negative integer, but is {self.top_k}")

    def check_vocab(self, vocab_size):
        if self.temp != 0 and self.top_k and not (0 < self.top_k < vocab_size):
            raise ValueError(
                f"`top_k` has to be an integer in the (0, {vocab_size}) interval, but is {self.top_k}."
            )

    @property
    def greedy(self):
        return self.temp == 0

    def __call__(self, logprobs):
        from .sampling import sample_batch

        if logprobs.dim() == 1:
            logprobs = logprobs[None]
        n = logprobs.shape[0]
        seed = self.seed if self.seed is not None else default_seed()
        tokens, _ = sample_batch(logprobs, [self] * n, seeds=[seed + i for i in range(n)],
                                 counters=[self._calls] * n)
        self._calls += 1
        return tokens.clone()  # the batch sampler's buffers are reused


def make_sampler(temp=0.0, top_p=0.0, min_p=0.0, min_tokens_to_keep=1, top_k=0, xtc_probability=0.0,
                 xtc_threshold=0.1, xtc_special_tokens=[]):
    """A sampler with the reference's options (mlx_lm/sample_utils.py:10-69)."""
    return Sampler(temp, top_p, min_p, min_tokens_to_keep, top_k, xtc_probability, xtc_threshold,
                   list(xtc_special_tokens))


_DEFAULT_SEED = [0]


def seed(value):
    """Seed for samplers that are given none (the reference's ``mx.random.seed``)."""
    _DEFAULT_SEED[0] = int(value)


def default_seed():
    return _DEFAULT_SEED[0]


# ---------------------------------------------------------------------------
# logits processors: callables (tokens, logits) -> logits


@dataclass
class LogitBias:
    """Adds ``bias[token]`` to the logits (mlx_lm/sample_utils.py:105-113)."""

    bias: Dict[int, float]

    def __call__(self, tokens, logits):
        from .sampling import apply_processors

        return apply_processors(logits, [[self]], [list(_as_list(tokens))])


@dataclass
class RepetitionPenalty:
    """Multiplicative, sign-aware penalty on tokens of the last ``context_size``
    (mlx_lm/sample_utils.py:284-315)."""

    penalty: float
    context_size: int = 20

    def __post_init__(self):
        if not isinstance(self.penalty, (int, float)) or self.penalty < 0:
            raise ValueError(f"penalty must be a non-negative float, got {self.penalty}")

    def __call__(self, tokens, logits):
        from .sampling import apply_processors

        return apply_processors(logits, [[self]], [list(_as_list(tokens))])


@dataclass
class PresencePenalty:
    """Subtracts ``penalty`` once for every token that occurs in the last
    ``context_size`` (mlx_lm/sample_utils.py:318-342)."""

    penalty: float
    context_size: int = 20

    __call__ = RepetitionPenalty.__call__


@dataclass
class FrequencyPenalty:
    """Subtracts ``penalty`` for every occurrence in the last ``context_size``
    (mlx_lm/sample_utils.py:345-369)."""

    penalty: float
    context_size: int = 20

    __call__ = RepetitionPenalty.__call__


def _as_list(tokens):
    if isinstance(tokens, torch.Tensor):
        return tokens.tolist()
    return list(tokens)


def make_logits_processors(logit_bias=None, repetition_penalty=None, repetition_context_size=20,
                           presence_penalty=None, presence_context_size=20, frequency_penalty=None,
                           frequency_context_size=20):
    """The reference's list of processors, in its order (mlx_lm/sample_utils.py:72-126)."""
    out = []
    if logit_bias:
        out.append(LogitBias({int(k): float(v) for k, v in logit_bias.items()}))
    if repetition_penalty is not None and repetition_penalty != 0:
        out.append(RepetitionPenalty(repetition_penalty, repetition_context_size))
    if presence_penalty is not None and presence_penalty != 0:
        out.append(PresencePenalty(presence_penalty, presence_context_size))
    if frequency_penalty is not None and frequency_penalty != 0:
        out.append(FrequencyPenalty(frequency_penalty, frequency_context_size))
    return out
