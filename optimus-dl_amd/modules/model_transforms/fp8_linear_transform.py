"""Model transform that swaps ``nn.Linear`` for :class:`FP8Linear`.

Registered under the reference's name ``"transformer_engine"`` (so existing
``model_transforms: [{_name: transformer_engine, ...}]`` YAML keeps working) and
under the native name ``"fp8_linear"``.  Behaviour follows
optimus_dl/modules/model_transforms/transformer_engine.py:

  * config keys and defaults of TransformerEngineTransformConfig (:362-398);
  * exact fully-qualified class-name match against a replacement table
    (:254-275, :334-354, :501-513) - subclasses of nn.Linear are left alone;
  * in-place ``setattr`` on the parent, the model object itself is returned
    (:556-558; tests assert identity); disabled or backend missing -> untouched
    (:447-449);
  * counters per kind and the two summary log lines (:454-476).

Deviations, on purpose:
  * the replacement shares the original ``Parameter`` objects instead of copying
    them (:278-290 copies, which unties ``lm_head`` from ``wte``);
  * ``replace_norm`` re-classes RMSNorm and LayerNorm modules in place (same object, same
    keys) so that their forward is the fused kernel that also feeds the next Linear's
    quantisation; ``replace_attention`` is accepted and ignored;
  * ``fuse_swiglu`` (an extra key, default on) does the same for SwiGLU MLPs whose three
    projections were converted: ``silu(w1 x) * w2 x`` becomes one kernel; ``fuse_gelu`` (likewise)
    for exact ``nn.GELU`` modules (the activation of the GPT-2 MLP);
  * a conversion that throws is logged at WARNING (the reference logs at DEBUG).
"""

from __future__ import annotations

import logging
from dataclasses import dataclass
from typing import Any, Callable

import torch.nn as nn

from ... import native
from ..fp8_linear import FP8Linear, SiblingGroup
from ..fused import fuse_gelu, fuse_layernorm, fuse_rmsnorm, fuse_swiglu_mlp
from . import register_model_transform
from .base import BaseModelTransform
from .config import ModelTransformConfig

logger = logging.getLogger(__name__)

_HAVE_TE = native.is_built()   # name kept so that code which patches / reads this flag keeps working


def is_transformer_engine_available() -> bool:
    return _HAVE_TE


TELinear = FP8Linear   # the reference's wrapper name

# fully-qualified class name -> (replacement class, converter, kind)
SUPPORTED_MODULE_REPLACEMENTS: dict[str, tuple[type, Callable[..., nn.Module] | None, str]] = {}


def _register_replacement(module_path: str, replacement_class: type, converter: Callable[..., nn.Module] | None = None,
                          module_type: str = "norm") -> None:
    SUPPORTED_MODULE_REPLACEMENTS[module_path] = (replacement_class, converter, module_type)


def _get_module_class_name(module: nn.Module) -> str:
    cls = module.__class__
    return f"{cls.__module__}.{cls.__name__}"


def _convert_linear(original: nn.Linear, **kwargs: Any) -> FP8Linear:
    return FP8Linear.from_linear(original, **kwargs)


_register_replacement("torch.nn.modules.linear.Linear", FP8Linear, _convert_linear, "linear")


def _convert_rmsnorm(original: nn.Module, **kwargs: Any) -> nn.Module | None:
    """In place: the module keeps its identity, parameters and keys; None if nothing changed."""
    return original if fuse_rmsnorm(original) else None


def _convert_layernorm(original: nn.Module, **kwargs: Any) -> nn.Module | None:
    return original if fuse_layernorm(original) else None


# the LayerNorm classes the reference's table names (transformer_engine.py:344-352)
for _path in ("optimus_dl.modules.model.blocks.layer_norms.LayerNorm", "torch.nn.modules.normalization.LayerNorm"):
    _register_replacement(_path, nn.Module, _convert_layernorm, "norm")

# the reference's RMSNorm (layer_norms.py:50) and the one of this package's own blocks
for _path in ("optimus_dl.modules.model.blocks.layer_norms.RMSNorm", "optimus_dl_amd.modules.model.blocks.RMSNorm",
              "optimus-dl_amd.modules.model.blocks.RMSNorm"):
    _register_replacement(_path, nn.Module, _convert_rmsnorm, "norm")


@dataclass
class TransformerEngineTransformConfig(ModelTransformConfig):
    enabled: bool = True
    replace_linear: bool = True
    replace_norm: bool = True          # RMSNorm / LayerNorm -> fused forward (in place)
    replace_attention: bool = False    # accepted, no effect here
    linear_kwargs: dict = None
    norm_kwargs: dict = None
    attention_kwargs: dict = None
    replace_inplace: bool = True
    verbose: bool = False
    fuse_swiglu: bool = True           # not in the reference: SwiGLU MLPs get the fused activation
    swiglu_classes: tuple = ("SwiGLUMLP",)
    fuse_gelu: bool = True             # not in the reference: exact nn.GELU modules get the fused activation
    # not in the reference: Linears of one parent that its forward feeds the same tensor (attention.py:317-319,
    # mlp.py:76-78) run as one autograd node whose data gradients the GEMMs sum themselves
    group_siblings: tuple = (("wq", "wk", "wv"), ("w1", "w2"))

    def __post_init__(self):
        self.linear_kwargs = dict(self.linear_kwargs or {})
        self.norm_kwargs = dict(self.norm_kwargs or {})
        self.attention_kwargs = dict(self.attention_kwargs or {})


Fp8LinearTransformConfig = TransformerEngineTransformConfig


@register_model_transform("fp8_linear", TransformerEngineTransformConfig)
@register_model_transform("transformer_engine", TransformerEngineTransformConfig)
class TransformerEngineTransform(BaseModelTransform):
    """nn.Linear -> FP8Linear over the whole module tree."""

    def __init__(self, cfg: TransformerEngineTransformConfig, **kwargs: Any):
        super().__init__(cfg, **kwargs)
        if not _HAVE_TE:
            logger.warning(
                "FP8 kernel library not built. The FP8 model transform will be a no-op. "
                "Build with: python -m optimus_dl_amd.build"
            )

    def apply(self, model: nn.Module, **kwargs: Any) -> nn.Module:
        if not self.cfg.enabled or not _HAVE_TE:
            logger.info("FP8 transform disabled or backend not available, skipping")
            return model
        logger.info("Applying FP8 module replacements")
        replacements = {"Linear": 0, "RMSNorm": 0, "LayerNorm": 0, "Attention": 0}
        self.sibling_groups = 0            # groups of Linears fed by one tensor (not module replacements: counted apart)
        self._replace_modules_recursive(model, replacements, replace_linear=self.cfg.replace_linear,
                                        replace_norm=self.cfg.replace_norm, replace_attention=self.cfg.replace_attention)
        total = sum(replacements.values())
        if self.cfg.verbose or total > 0:
            logger.info(f"TE module replacements: {replacements}")
            logger.info(f"Total modules replaced: {total}")
        self.last_replacements = replacements
        return model

    def _pick(self, module_type: str, class_name: str, replace_linear: bool, replace_norm: bool, replace_attention: bool):
        if module_type == "linear":
            return replace_linear, self.cfg.linear_kwargs, "Linear"
        if module_type == "norm":
            return replace_norm, self.cfg.norm_kwargs, "RMSNorm" if "RMSNorm" in class_name else "LayerNorm"
        if module_type == "attention":
            return replace_attention, self.cfg.attention_kwargs, "Attention"
        return False, {}, None

    def _replace_modules_recursive(self, module: nn.Module, replacements: dict[str, int], replace_linear: bool,
                                   replace_norm: bool, replace_attention: bool, parent: nn.Module | None = None,
                                   name: str | None = None) -> None:
        entry = SUPPORTED_MODULE_REPLACEMENTS.get(_get_module_class_name(module))
        if entry is not None:
            replacement_class, converter, module_type = entry
            enabled, mod_kwargs, key = self._pick(module_type, module.__class__.__name__, replace_linear, replace_norm,
                                                  replace_attention)
            if enabled and module_type == "norm" and not self.cfg.replace_inplace:
                enabled = False            # the norm conversion only exists in place
            if enabled:
                try:
                    new_module = converter(module, **mod_kwargs) if converter else replacement_class(**module.__dict__)
                except Exception as e:  # a layer that cannot be converted stays as it is
                    logger.warning(f"Failed to replace {_get_module_class_name(module)}: {e}")
                    new_module = None
                if new_module is not None:
                    replacements[key] = replacements.get(key, 0) + 1
                    if self.cfg.replace_inplace and parent is not None and name is not None:
                        setattr(parent, name, new_module)
                    elif self.cfg.verbose:
                        logger.debug(f"Would replace {_get_module_class_name(module)} with {type(new_module)}")
        for child_name, child in list(module.named_children()):
            self._replace_modules_recursive(child, replacements, replace_linear, replace_norm, replace_attention,
                                            parent=module, name=child_name)
        if self.cfg.fuse_gelu and self.cfg.replace_inplace and _get_module_class_name(module) == "torch.nn.modules.activation.GELU" \
                and fuse_gelu(module):
            replacements["GELU"] = replacements.get("GELU", 0) + 1
        if self.cfg.replace_inplace:
            for names in tuple(self.cfg.group_siblings or ()):
                members = [getattr(module, n, None) for n in names]
                if all(isinstance(m, FP8Linear) for m in members) and len({id(m) for m in members}) == len(members) \
                        and len({m.in_features for m in members}) == 1 and not any(m._siblings is not None for m in members):
                    SiblingGroup(members)
                    self.sibling_groups += 1
        # after the children: the three projections of an MLP are FP8 Linears by now
        if (self.cfg.fuse_swiglu and self.cfg.replace_inplace and module.__class__.__name__ in tuple(self.cfg.swiglu_classes)
                and fuse_swiglu_mlp(module)):
            replacements["SwiGLU"] = replacements.get("SwiGLU", 0) + 1


Fp8LinearTransform = TransformerEngineTransform
