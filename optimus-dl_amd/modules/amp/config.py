"""Re-export of the AMP config dataclasses (optimus_dl/modules/amp/config.py:7-11)."""
from ..optim.config import AmpConfig, Fp8Config, OptimizationConfig

__all__ = ["AmpConfig", "Fp8Config", "OptimizationConfig"]
