"""Model-transform registry (optimus_dl/modules/model_transforms/__init__.py:7-9)."""
from ...core.registry import make_registry
from .base import BaseModelTransform
from .config import ModelTransformConfig

_MODEL_TRANSFORMS_REGISTRY, register_model_transform, build_model_transform = make_registry("model_transform")

from . import fp8_linear_transform  # noqa: E402,F401  (registers "transformer_engine" and "fp8_linear")

__all__ = ["BaseModelTransform", "ModelTransformConfig", "register_model_transform", "build_model_transform"]
