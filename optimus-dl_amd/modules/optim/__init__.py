from .config import AmpConfig, Fp8Config, OptimizationConfig

__all__ = ["AmpConfig", "Fp8Config", "OptimizationConfig"]
