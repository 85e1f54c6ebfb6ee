"""What an architecture is made of, as data.

An architecture's arguments are turned into a ``ModelPlan``: which part (by
registry key, with its sizes and constants as parameters and the prefix of its
tensor names) sits where in each layer, and in which order layers run.  The
builder in ``parts.model`` makes the parts from the plan; nothing in a part
names the architecture it is used in.
"""

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


@dataclass(frozen=True)
class PartSpec:
    """One part: registry key, constructor parameters, tensor-name prefix."""

    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    prefix: str = ""


@dataclass(frozen=True)
class LayerSpec:
    """One layer: an arrangement (block kind) and the parts it arranges, by the names
    that the arrangement gives them (``pre_norm``: ``mixer_norm``, ``mixer``, ``ffn_norm``,
    ``ffn``).  Which parts there are, and how many, is the arrangement's business."""

    arrangement: str
    parts: Dict[str, PartSpec]


@dataclass(frozen=True)
class RunEntry:
    """One run of a layer.

    ``layer`` indexes ``ModelPlan.layers`` and may occur more than once in the
    schedule.  ``cache`` names the cache slot that this run's mixer reads; two
    runs that name the same slot share keys and values, and only the run with
    ``writes_cache`` puts this step's tokens there (it has to come first).
    """

    layer: int
    cache: int
    writes_cache: bool = True


@dataclass(frozen=True)
class CacheNeed:
    """Paged keys and values that a mixer wants for one cache slot."""

    n_kv_heads: int
    head_dim: int  # width of a head's key
    window: int = 0  # 0: every earlier token; n: the last n tokens
    v_head_dim: int = 0  # width of a head's value; 0: as the key's

    @property
    def value_dim(self):
        return self.v_head_dim or self.head_dim


@dataclass(frozen=True)
class StateNeed:
    """Per-request state of fixed size that a mixer wants for one cache slot."""

    shape: Tuple[int, ...]
    dtype: str = "float32"


@dataclass
class ModelPlan:
    width: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    embedding_positions: Optional[PartSpec]
    layers: List[LayerSpec]
    schedule: List[RunEntry]
    final_norm: PartSpec
    head: PartSpec

    def validate(self):
        n_layers = len(self.layers)
        written = set()
        for i, run in enumerate(self.schedule):
            if not (0 <= run.layer < n_layers):
                raise ValueError(f"schedule entry {i} names layer {run.layer}, there are {n_layers}")
            if run.writes_cache:
                if run.cache in written:
                    raise ValueError(f"schedule entry {i}: cache slot {run.cache} is written twice")
                written.add(run.cache)
            elif run.cache not in written:
                raise ValueError(
                    f"schedule entry {i} reads cache slot {run.cache} before any run has written it"
                )
        slots = sorted(written)
        if slots != list(range(len(slots))):
            raise ValueError(f"cache slots must be numbered 0..n-1 without gaps, got {slots}")
        return self

    @property
    def n_cache_slots(self):
        return len({run.cache for run in self.schedule})
