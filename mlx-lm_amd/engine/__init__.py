"""The step function, the scheduler above it, and trace replay."""

from .step import Engine, StepEntry

__all__ = ["Engine", "StepEntry"]
