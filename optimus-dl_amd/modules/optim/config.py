"""AMP / FP8 configuration surface (keys and defaults of
optimus_dl/modules/optim/config.py:17-130, which the YAML groups
configs/train/optimization/amp/fp8_{hybrid,e4m3}.yaml fill in).

Keys the reference declares but never reads (param, wgrad, first_last_layers_bf16,
num_layers_at_*_in_bf16, tp_only_amax_red) are accepted; ``wgrad=False`` is
honoured here (weight gradients in bf16), ``param`` and ``first_last_layers_bf16`` act through
``TrainingContext.attach_fp8_params`` / ``apply_fp8_layer_policy``, ``tp_only_amax_red`` is carried through.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass
class Fp8Config:
    enabled: bool = False
    format: str = "hybrid"            # hybrid | e4m3 | e5m2
    recipe: str = "delayed"           # delayed | tensorwise | blockwise | mxfp8 (+ rowwise, an extension)
    param: bool = False
    margin: int = 0
    amax_history_len: int = 1024
    amax_compute_algo: str = "max"    # max | most_recent
    reduce_amax: bool = True
    wgrad: bool = True
    fp8_dpa: bool = False
    fp8_mha: bool = False
    first_last_layers_bf16: bool = False
    num_layers_at_start_in_bf16: int = 1
    num_layers_at_end_in_bf16: int = 1
    tp_only_amax_red: bool = False


@dataclass
class AmpConfig:
    enabled: bool = False
    dtype: str = "torch.bfloat16"
    # The reference leaves this to a config-time expression ("fp16 => True");
    # None means exactly that rule, resolved in resolved_enable_scaler().
    enable_scaler: Any = None
    init_scale: float = 2.0**16
    growth_factor: float = 2.0
    backoff_factor: float = 0.5
    growth_interval: int = 2000
    fp8: Fp8Config = field(default_factory=Fp8Config)

    def __post_init__(self) -> None:
        if isinstance(self.fp8, dict):
            self.fp8 = Fp8Config(**self.fp8)

    def resolved_enable_scaler(self) -> bool:
        if isinstance(self.enable_scaler, bool):
            return self.enable_scaler
        if isinstance(self.enable_scaler, str) and self.enable_scaler.strip().lower() in ("true", "false"):
            return self.enable_scaler.strip().lower() == "true"
        return str(self.dtype) in ("torch.float16", "float16", "fp16", "half")


@dataclass
class OptimizationConfig:
    optimizer: Any = None
    iterations: int = 1000
    acc_steps: int = 1
    clip_grad_norm: float | None = None
    amp: AmpConfig = field(default_factory=AmpConfig)

    def __post_init__(self) -> None:
        if isinstance(self.amp, dict):
            self.amp = AmpConfig(**self.amp)
