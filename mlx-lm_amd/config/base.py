"""Base of every architecture's typed arguments."""

import inspect
from dataclasses import dataclass


@dataclass
class BaseModelArgs:
    """A dataclass of config.json keys.

    ``from_dict`` keeps the keys that are constructor parameters and drops the
    rest, as the reference does (mlx_lm/models/base.py:11-21); what a subclass
    cannot run it refuses in its ``__post_init__``.
    """

    @classmethod
    def from_dict(cls, params):
        names = inspect.signature(cls).parameters
        return cls(**{k: v for k, v in params.items() if k in names})
