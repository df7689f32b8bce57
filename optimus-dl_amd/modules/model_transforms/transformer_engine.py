"""Import-path compatibility: the reference keeps this transform in
``modules/model_transforms/transformer_engine.py``; the implementation here lives
in ``fp8_linear_transform.py``."""
from .fp8_linear_transform import (  # noqa: F401
    SUPPORTED_MODULE_REPLACEMENTS,
    TELinear,
    TransformerEngineTransform,
    TransformerEngineTransformConfig,
    _convert_linear,
    _get_module_class_name,
    _register_replacement,
    is_transformer_engine_available,
)
