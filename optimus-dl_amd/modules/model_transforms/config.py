from dataclasses import dataclass

from ...core.registry import RegistryConfig


@dataclass
class ModelTransformConfig(RegistryConfig):
    """Base config of model transforms (open: unknown keys are tolerated)."""
