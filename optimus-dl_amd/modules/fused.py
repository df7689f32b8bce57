"""Producers either side of the FP8 Linear that hand their output's partial maxima to it.

The reference leaves these to PyTorch: ``silu(w1(x)) * w2(x)`` in
optimus_dl/modules/model/blocks/mlp.py:73-76 and RMSNorm in
optimus_dl/modules/model/blocks/layer_norms.py:86-119.  Here one kernel writes the bf16
result and, on the way, the partial maxima of its magnitude; the FP8 Linear that consumes
that very tensor finds them (``FP8Recipe.take_parts``) and casts without an amax pass.
Modules are not replaced but re-classed in place (``module.__class__`` becomes a subclass of
its own class with the forward below), so attributes, parameter names, state-dict keys and
``isinstance`` checks stay what they were.

Without an active FP8 recipe, on the CPU, or for dtypes the kernels do not take, every
forward below is the module's own.
"""

from __future__ import annotations

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import native
from .amp import state as _state
from .amp.fp8 import FP8Recipe
from .fp8_linear import FP8Linear


def _bf16_cuda(*tensors: torch.Tensor) -> bool:
    return all(t.is_cuda and t.dtype == torch.bfloat16 for t in tensors)


# ------------------------------------------------------------------------- SwiGLU
class _SwiGLUFn(torch.autograd.Function):
    """h = silu(gate) * up with the roundings of eager bf16 arithmetic; gate and up are kept for
    the backward, h is not (the down projection keeps its FP8 codes only)."""

    @staticmethod
    def forward(ctx, gate: torch.Tensor, up: torch.Tensor, recipe: FP8Recipe):
        h, parts = native.swiglu_amax_parts(gate, up)
        recipe.offer_parts(h, parts)
        ctx.save_for_backward(gate, up)
        ctx.recipe = recipe
        return h

    @staticmethod
    def backward(ctx, dh: torch.Tensor):
        gate, up = ctx.saved_tensors
        if dh.dtype != torch.bfloat16:
            dh = dh.to(torch.bfloat16)
        dgate, dup, parts_g, parts_u = native.swiglu_bwd_amax_parts(dh, gate, up)
        ctx.recipe.offer_parts(dgate, parts_g)
        ctx.recipe.offer_parts(dup, parts_u)
        return dgate, dup, None


@torch.compiler.disable
def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up; fused (and feeding the next FP8 Linear) when an FP8 recipe is active."""
    recipe = _state.active_recipe()
    if recipe is None or not _bf16_cuda(gate, up) or gate.shape != up.shape or gate.numel() % 8:
        return F.silu(gate) * up
    return _SwiGLUFn.apply(gate, up, recipe)


# ---------------------------------------------------------------- in-place re-classing
# A module is fused by giving it a subclass of its own class with the fused forward mixed in: same object, same
# parameters, same state-dict keys, isinstance() checks keep working.  The subclass is made on the fly, so pickling
# it by name would find the original class instead: the mixins carry a __reduce_ex__ that rebuilds the subclass
# from (original class, mixin) -- copy.deepcopy (EMA copies of a model) and torch.save of a whole module both work.
_RECLASSED: dict[tuple[type, type], type] = {}


def _fused_class(base: type, mixin: type) -> type:
    key = (base, mixin)
    cls = _RECLASSED.get(key)
    if cls is None:
        cls = type(base.__name__, (mixin, base), {"__module__": base.__module__})
        _RECLASSED[key] = cls
    return cls


def _rebuild_fused(base: type, mixin: type):
    cls = _fused_class(base, mixin)
    return cls.__new__(cls)


class _Reclassed:
    def __reduce_ex__(self, protocol):
        mro = type(self).__mro__                      # (made-up subclass, mixin, _Reclassed, original class, ...)
        return _rebuild_fused, (mro[mro.index(_Reclassed) + 1], mro[1]), self.__dict__


class _FusedSwiGLUForward(_Reclassed):
    """Mixed into the class of an MLP with ``w1`` (gate), ``w2`` (up) and ``c_proj`` (down)."""

    _odl_fused_swiglu = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if _state.active_recipe() is None or not x.is_cuda:
            return super().forward(x)
        return self.c_proj(swiglu(self.w1(x), self.w2(x)))


def fuse_swiglu_mlp(mlp: nn.Module) -> bool:
    """Re-class ``mlp`` in place so that its forward is the fused one.  Only modules whose three
    projections are FP8 Linears named as in the reference's SwiGLUMLP (mlp.py:47-49) qualify."""
    if getattr(mlp, "_odl_fused_swiglu", False):
        return False
    if not all(isinstance(getattr(mlp, n, None), FP8Linear) for n in ("w1", "w2", "c_proj")):
        return False
    cls = mlp.__class__
    mlp.__class__ = _fused_class(cls, _FusedSwiGLUForward)
    return True


# ------------------------------------------------------------------------ RMSNorm
class _RMSNormFn(torch.autograd.Function):
    """y = (x * rsqrt(mean(x^2) + eps)) * weight rounded once to bf16."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, weight: torch.Tensor, eps: float, recipe: FP8Recipe):
        y, rstd, parts = native.rmsnorm_amax_parts(x, weight, eps)
        recipe.offer_parts(y, parts)
        ctx.save_for_backward(x, weight, rstd)
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        x, weight, rstd = ctx.saved_tensors
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        dx, dw = native.rmsnorm_bwd(dy, x, weight, rstd)
        return (dx if ctx.needs_input_grad[0] else None), (dw.to(weight.dtype) if ctx.needs_input_grad[1] else None), None, None


@torch.compiler.disable
def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor | None:
    """Fused RMSNorm when an FP8 recipe is active and the kernel takes the input; else None."""
    recipe = _state.active_recipe()
    if recipe is None or not x.is_cuda or x.dtype not in (torch.bfloat16, torch.float32):
        return None
    if x.dtype != torch.bfloat16 and not (torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") == torch.bfloat16):
        return None                    # an fp32 result is expected downstream: the module's own forward
    cols = x.shape[-1]
    if cols % 8 or cols < 8 or cols > 8192 or weight.numel() != cols or x.numel() == 0:
        return None
    return _RMSNormFn.apply(x, weight, float(eps), recipe)


class _FusedRMSNormForward(_Reclassed):
    """Mixed into the class of an RMSNorm with ``weight`` and ``eps`` (layer_norms.py:64-67).

    Under an FP8 recipe the output is bf16 whatever the input dtype: the recipe's context nests
    a bf16 autocast (fp8.py:488-493), so the Linear that follows would round an fp32 output to
    bf16 anyway; the values are the same, the fp32 copy is never written."""

    _odl_fused_rmsnorm = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = rmsnorm(x, self.weight, self.eps)
        return super().forward(x) if y is None else y


def fuse_rmsnorm(norm: nn.Module) -> bool:
    if getattr(norm, "_odl_fused_rmsnorm", False):
        return False
    w = getattr(norm, "weight", None)
    if not isinstance(w, torch.Tensor) or w.dim() != 1 or not hasattr(norm, "eps"):
        return False
    cls = norm.__class__
    norm.__class__ = _fused_class(cls, _FusedRMSNormForward)
    return True


# ---------------------------------------------------------------------- LayerNorm
class _LayerNormFn(torch.autograd.Function):
    """y = layer_norm(x) * weight + bias rounded once to bf16."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, eps: float, recipe: FP8Recipe):
        y, mean, rstd, parts = native.layernorm_amax_parts(x, weight, bias, eps)
        recipe.offer_parts(y, parts)
        ctx.save_for_backward(x, weight, mean, rstd)
        ctx.bias_dtype = None if bias is None else bias.dtype
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        x, weight, mean, rstd = ctx.saved_tensors
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        dx, dw, db = native.layernorm_bwd(dy, x, weight, mean, rstd)
        return (dx if ctx.needs_input_grad[0] else None, dw.to(weight.dtype) if ctx.needs_input_grad[1] else None,
                db.to(ctx.bias_dtype) if ctx.bias_dtype is not None and ctx.needs_input_grad[2] else None, None, None)


@torch.compiler.disable
def layernorm(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, eps: float) -> torch.Tensor | None:
    """Fused LayerNorm when an FP8 recipe is active and the kernel takes the input; else None."""
    recipe = _state.active_recipe()
    if recipe is None or not x.is_cuda or x.dtype not in (torch.bfloat16, torch.float32):
        return None
    if x.dtype != torch.bfloat16 and not (torch.is_autocast_enabled("cuda") and torch.get_autocast_dtype("cuda") == torch.bfloat16):
        return None
    cols = x.shape[-1]
    if cols % 8 or cols < 8 or cols > 4096 or weight is None or weight.numel() != cols or x.numel() == 0:
        return None
    return _LayerNormFn.apply(x, weight, bias, float(eps), recipe)


class _FusedLayerNormForward(_Reclassed):
    """Mixed into the class of a LayerNorm over the last axis: ``torch.nn.LayerNorm`` (``normalized_shape``
    of one dimension, affine) or the reference's bias-optional one (layer_norms.py:21-47, eps 1e-5).
    Output dtype under an FP8 recipe: as for the fused RMSNorm."""

    _odl_fused_layernorm = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = layernorm(x, self.weight, getattr(self, "bias", None), getattr(self, "eps", 1e-5))
        return super().forward(x) if y is None else y


def fuse_layernorm(norm: nn.Module) -> bool:
    if getattr(norm, "_odl_fused_layernorm", False):
        return False
    w = getattr(norm, "weight", None)
    if not isinstance(w, torch.Tensor) or w.dim() != 1:
        return False                       # no affine weight, or normalisation over several axes
    shape = getattr(norm, "normalized_shape", None)
    if shape is not None and tuple(shape) != (w.numel(),):
        return False
    cls = norm.__class__
    norm.__class__ = _fused_class(cls, _FusedLayerNormForward)
    return True


# --------------------------------------------------------------------------- GELU
class _GeluFn(torch.autograd.Function):
    """Exact (erf) GELU of a bf16 tensor, its input kept for the backward."""

    @staticmethod
    def forward(ctx, x: torch.Tensor, recipe: FP8Recipe):
        y, parts = native.gelu_amax_parts(x)
        recipe.offer_parts(y, parts)
        ctx.save_for_backward(x)
        ctx.recipe = recipe
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        (x,) = ctx.saved_tensors
        if dy.dtype != torch.bfloat16:
            dy = dy.to(torch.bfloat16)
        dx, parts = native.gelu_bwd_amax_parts(dy, x)
        ctx.recipe.offer_parts(dx, parts)
        return dx, None


@torch.compiler.disable
def gelu(x: torch.Tensor) -> torch.Tensor | None:
    """Fused GELU when an FP8 recipe is active and the input is a bf16 GPU tensor; else None."""
    recipe = _state.active_recipe()
    if recipe is None or not _bf16_cuda(x) or x.numel() % 8 or x.numel() == 0:
        return None
    return _GeluFn.apply(x, recipe)


class _FusedGeluForward(_Reclassed):
    """Mixed into the class of an ``nn.GELU`` with the exact (erf) form, the activation of the
    reference's GELUMLP (mlp.py:141-157)."""

    _odl_fused_gelu = True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        y = gelu(x)
        return super().forward(x) if y is None else y


def fuse_gelu(act: nn.Module) -> bool:
    if getattr(act, "_odl_fused_gelu", False) or not isinstance(act, nn.GELU) or getattr(act, "approximate", "none") != "none":
        return False
    cls = act.__class__
    act.__class__ = _fused_class(cls, _FusedGeluForward)
    return True
