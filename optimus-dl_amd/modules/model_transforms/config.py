"""Import location kept for callers that take the transform options from here, as
with optimus_dl/modules/model_transforms/config.py; the class is defined beside the
transform base class."""

from .base import ModelTransformConfig

__all__ = ["ModelTransformConfig"]
