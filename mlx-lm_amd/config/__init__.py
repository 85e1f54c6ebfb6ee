"""Typed configuration: per-architecture argument classes, the plan that an
architecture turns them into, and the registry from ``model_type`` to both."""

from .base import BaseModelArgs
from .plan import CacheNeed, LayerSpec, ModelPlan, PartSpec, RunEntry, StateNeed
from .registry import MODEL_REMAPPING, get_model_classes, register_model, registered_model_types

__all__ = [
    "BaseModelArgs",
    "CacheNeed",
    "StateNeed",
    "LayerSpec",
    "ModelPlan",
    "PartSpec",
    "RunEntry",
    "MODEL_REMAPPING",
    "get_model_classes",
    "register_model",
    "registered_model_types",
]
