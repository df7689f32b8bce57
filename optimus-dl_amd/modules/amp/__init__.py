"""AMP package facade (same public names as optimus_dl/modules/amp/__init__.py:46-64)."""
from .config import AmpConfig, Fp8Config, OptimizationConfig
from .fp8 import (
    FP8Recipe,
    Fp8Format,
    Fp8RecipeConfig,
    Fp8RecipeType,
    ScalingPolicy,
    create_fp8_recipe,
    fp8_autocast,
    fp8_backward,
    get_fp8_format_from_string,
    get_fp8_recipe_type_from_string,
    get_transformer_engine_version,
    is_native_backend_available,
    is_transformer_engine_available,
)

__all__ = [
    "AmpConfig", "Fp8Config", "OptimizationConfig", "FP8Recipe", "Fp8Format", "Fp8RecipeConfig", "Fp8RecipeType",
    "ScalingPolicy", "create_fp8_recipe", "fp8_autocast", "fp8_backward", "get_fp8_format_from_string",
    "get_fp8_recipe_type_from_string", "get_transformer_engine_version", "is_native_backend_available",
    "is_transformer_engine_available",
]
