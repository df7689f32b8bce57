"""The callers of the FP8 path inside a training loop.

``TrainingContext.setup_training_context`` reproduces the decision table of
optimus_dl/recipe/train/mixins/execution/context_mixin.py:49-149 (is the AMP
dtype an FP8 dtype? is the device "cuda"? is the backend there? is
``amp.fp8.enabled`` set?) and returns the same 8-key dict.
``execute_forward_pass`` / ``execute_backward_pass`` follow
.../iteration_mixin.py:101-185: ``amp_ctx`` and ``fp8_backward_ctx`` may be a
context-manager instance or a zero-argument factory, re-entered every microbatch.
``forward_context`` is the evaluation-side wrapper
(.../managers/evaluation_manager.py:98-144): FP8 autocast with bf16 inside, on the
scales the training steps measured.
"""

from __future__ import annotations

import logging
from contextlib import contextmanager, nullcontext
from typing import Any

import torch

from ..core.dtype import get_fp8_format_from_dtype, is_fp8_dtype, str_to_dtype
from ..modules.amp.fp8 import (
    FP8Recipe,
    create_fp8_recipe,
    fp8_autocast,
    is_transformer_engine_available,
)
from ..modules.optim.config import AmpConfig, OptimizationConfig

logger = logging.getLogger(__name__)


class TrainingContext:
    def __init__(self, optimization_config: OptimizationConfig):
        self.optimization_config = optimization_config
        self._fp8_recipe: FP8Recipe | None = None

    def setup_training_context(self, device: torch.device) -> dict[str, Any]:
        amp_cfg: AmpConfig = self.optimization_config.amp
        dtype = str_to_dtype(amp_cfg.dtype)
        is_fp8 = is_fp8_dtype(dtype)
        if is_fp8:
            logger.info(f"FP8 format detected: {get_fp8_format_from_dtype(dtype)}")
        if is_fp8 and device.type != "cuda":
            raise ValueError("FP8 training is only supported on CUDA devices.")

        # FP8 scales its own tensors: no loss scaler
        enable_scaler = amp_cfg.resolved_enable_scaler() and not is_fp8
        scaler = torch.GradScaler(device=device.type, enabled=amp_cfg.enabled and enable_scaler,
                                  init_scale=amp_cfg.init_scale, growth_factor=amp_cfg.growth_factor,
                                  backoff_factor=amp_cfg.backoff_factor, growth_interval=amp_cfg.growth_interval)
        logger.info(f"Using grad scaler: {scaler.is_enabled()}")

        fp8_recipe, fp8_enabled = None, False
        if is_fp8 and amp_cfg.enabled and amp_cfg.fp8.enabled:
            if not is_transformer_engine_available():
                logger.warning("FP8 training requested but the FP8 backend is not available. "
                               "Falling back to standard AMP.")
            else:
                f = amp_cfg.fp8
                fp8_recipe = create_fp8_recipe(recipe_type=f.recipe, format=f.format, margin=f.margin,
                                               amax_history_len=f.amax_history_len,
                                               amax_compute_algo=f.amax_compute_algo, reduce_amax=f.reduce_amax,
                                               fp8_dpa=f.fp8_dpa, fp8_mha=f.fp8_mha, wgrad=f.wgrad)
                fp8_enabled = fp8_recipe is not None
                self._fp8_recipe = fp8_recipe

        if fp8_enabled and device.type == "cuda":
            amp_ctx = self._create_fp8_autocast(device, fp8_recipe)
        else:
            autocast_dtype = dtype
            if is_fp8 and amp_cfg.enabled:
                if device.type == "cuda" and torch.cuda.is_bf16_supported():
                    autocast_dtype = torch.bfloat16
                elif device.type == "cpu":
                    autocast_dtype = torch.bfloat16
                else:
                    autocast_dtype = torch.float16
                logger.info(f"Falling back from FP8 to standard AMP with dtype={autocast_dtype}")
            amp_ctx = torch.autocast(device.type, dtype=autocast_dtype, enabled=amp_cfg.enabled)

        return {
            "scaler": scaler,
            "amp_ctx": amp_ctx,
            "amp_cfg": amp_cfg,
            "device": device,
            "fp8_recipe": fp8_recipe,
            "fp8_enabled": fp8_enabled,
            "is_fp8_dtype": is_fp8,
            "fp8_backward_ctx": self.get_fp8_backward_ctx(),
        }

    def attach_fp8_params(self, model: torch.nn.Module, optimizer: "torch.optim.Optimizer | None" = None):
        """``amp.fp8.param: true``: the weights of the model's FP8 Linears stay quantised between optimizer steps
        (all of them re-quantised in one or two launches after each step).  Call once, after ``setup_training_context``
        and after model and optimizer exist.  Returns the parameter set, or None when the key is off, FP8 is not
        in use, or the recipe (rowwise) keeps the per-module route.  The reference declares the key and never reads it
        (optimus_dl/modules/optim/config.py:36-37,56)."""
        if self._fp8_recipe is None or not self.optimization_config.amp.fp8.param:
            return None
        return self._fp8_recipe.attach_params(model, optimizer)

    def apply_fp8_layer_policy(self, model: torch.nn.Module) -> list[str]:
        """``amp.fp8.first_last_layers_bf16: true``: the FP8 Linears of the model's first
        ``num_layers_at_start_in_bf16`` and last ``num_layers_at_end_in_bf16`` blocks run in the autocast dtype
        (optimus_dl/modules/optim/config.py:44-49,62-66; the reference declares the keys and never reads them).  Call
        once, after the model transform and before ``attach_fp8_params``.  Returns the names of the Linears kept out of
        FP8 (empty when the key is off or FP8 is not in use)."""
        fp8 = self.optimization_config.amp.fp8
        if self._fp8_recipe is None or not fp8.first_last_layers_bf16:
            return []
        from ..modules.fp8_linear import keep_layers_in_bf16

        return keep_layers_in_bf16(model, fp8.num_layers_at_start_in_bf16, fp8.num_layers_at_end_in_bf16)

    def _create_fp8_autocast(self, device: torch.device, fp8_recipe: FP8Recipe | None) -> Any:
        if fp8_recipe is not None:
            return lambda: fp8_autocast(device=device, fp8_recipe=fp8_recipe)   # a fresh context per microbatch
        return nullcontext()

    def get_fp8_backward_ctx(self) -> Any:
        if self._fp8_recipe is not None:
            return self._fp8_recipe.backward                                     # bound method = factory
        return nullcontext()


def _enter(ctx_or_factory: Any):
    """Accept a context manager or a zero-argument factory of one."""
    if ctx_or_factory is None:
        return nullcontext()
    if hasattr(ctx_or_factory, "__enter__"):
        return ctx_or_factory
    if callable(ctx_or_factory):
        return ctx_or_factory()
    return nullcontext()


def execute_forward_pass(model, batch, criterion, amp_ctx) -> torch.Tensor:
    with _enter(amp_ctx):
        return criterion(model, batch)


def execute_backward_pass(loss: torch.Tensor, scaler=None, fp8_backward_ctx=None) -> None:
    with _enter(fp8_backward_ctx):
        if scaler is not None and scaler.is_enabled():
            scaler.scale(loss).backward()
        else:
            loss.backward()


_eval_recipes: dict[tuple, FP8Recipe] = {}


def _eval_recipe(f) -> FP8Recipe | None:
    """The recipe of an evaluation forward.  The reference builds a new recipe object on every call
    (evaluation_manager.py:126-135); a recipe here carries no scaling state of its own (that lives with
    the modules), so one object per distinct configuration is kept and handed out again."""
    key = (str(f.recipe).lower(), str(f.format).lower(), f.margin, f.amax_history_len, f.amax_compute_algo, f.reduce_amax,
           f.fp8_dpa, f.fp8_mha)
    recipe = _eval_recipes.get(key)
    if recipe is None:
        recipe = create_fp8_recipe(recipe_type=f.recipe, format=f.format, margin=f.margin,
                                   amax_history_len=f.amax_history_len, amax_compute_algo=f.amax_compute_algo,
                                   reduce_amax=f.reduce_amax, fp8_dpa=f.fp8_dpa, fp8_mha=f.fp8_mha)
        if recipe is not None:
            _eval_recipes[key] = recipe
    return recipe


@contextmanager
def forward_context(amp_cfg: AmpConfig, device: torch.device):
    """Evaluation forward (evaluation_manager.py:98-144): nothing when AMP is off; FP8 autocast with bf16
    inside when the AMP dtype is an FP8 dtype, ``fp8.enabled`` is set and the backend is there; ordinary
    autocast otherwise (bf16 standing in for an FP8 dtype).  Modules in eval mode use the delayed-scaling
    scales that training measured and leave the amax histories alone."""
    if not amp_cfg.enabled:
        yield
        return
    dtype = str_to_dtype(amp_cfg.dtype)
    is_fp8 = is_fp8_dtype(dtype)
    recipe = None
    if is_fp8 and getattr(amp_cfg, "fp8", None) and amp_cfg.fp8.enabled and is_transformer_engine_available():
        recipe = _eval_recipe(amp_cfg.fp8)
    with fp8_autocast(device=device, fp8_recipe=recipe, enabled=True, dtype=torch.bfloat16 if is_fp8 else dtype):
        yield
