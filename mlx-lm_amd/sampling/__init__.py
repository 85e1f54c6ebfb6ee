"""Batched sampling on the GPU: one kernel launch for all rows of a step."""

from .sampler import PendingRead, SamplerBuffers, apply_processors, read_sampled, sample_batch

__all__ = ["PendingRead", "SamplerBuffers", "apply_processors", "read_sampled", "sample_batch"]
