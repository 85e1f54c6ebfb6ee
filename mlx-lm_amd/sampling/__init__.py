"""Batched sampling on the GPU: one kernel launch for all rows of a step."""

from .sampler import apply_processors, sample_batch

__all__ = ["apply_processors", "sample_batch"]
