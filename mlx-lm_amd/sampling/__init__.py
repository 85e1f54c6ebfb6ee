"""Batched sampling on the GPU: one kernel launch for all rows of a step."""

from .sampler import PendingRead, apply_processors, read_sampled, sample_batch

__all__ = ["PendingRead", "apply_processors", "read_sampled", "sample_batch"]
