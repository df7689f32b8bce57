"""Base class of model transforms (plugin API of
optimus_dl/modules/model_transforms/base.py:25-45): ``__init__(cfg, **kwargs)``
and ``apply(model, **kwargs) -> model``."""

from __future__ import annotations

from abc import ABC, abstractmethod
from dataclasses import dataclass
from typing import Any

import torch.nn as nn

from ...core.registry import RegistryConfig


@dataclass
class ModelTransformConfig(RegistryConfig):
    """Options every model transform accepts (the role of
    optimus_dl/modules/model_transforms/config.py:7-12).  It adds no field of its own:
    ``_name`` selects the transform in the registry, and keys a subclass does not
    declare are kept rather than rejected, so one YAML block can carry options for
    transforms this build does not have."""


class BaseModelTransform(ABC):
    def __init__(self, cfg: Any = None, **kwargs: Any):
        self.cfg = cfg

    @abstractmethod
    def apply(self, model: nn.Module, **kwargs: Any) -> nn.Module:
        """Return the transformed model (possibly the same object, modified in place)."""

    def __repr__(self) -> str:
        return f"{type(self).__name__}(cfg={self.cfg})"
