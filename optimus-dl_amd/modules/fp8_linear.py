"""FP8Linear: an ``nn.Linear`` whose matmuls run as FP8 MFMA GEMMs on MI355X.

Stands in for the reference's ``TELinear`` wrapper
(optimus_dl/modules/model_transforms/transformer_engine.py:63-111), which nests
a third-party ``te.pytorch.Linear``.  Differences that matter to callers:

  * it IS an ``nn.Linear`` (subclass) and, when made from an existing layer,
    keeps the very same ``Parameter`` objects.  State-dict keys stay
    ``<name>.weight`` / ``<name>.bias`` (the reference's wrapper renames them to
    ``<name>._te_linear.weight``), weight tying (``lm_head`` <-> ``wte``) survives,
    and code that selects parameters with ``isinstance(m, nn.Linear)`` keeps working;
  * outside an FP8 autocast context, on CPU, or for shapes the kernels cannot
    take (features or tokens not multiples of 16) it behaves as a plain Linear.

Per call, inside ``FP8Recipe.autocast()``:

  forward   Y  = Q(X)  . Q(W)^T      X, W -> E4M3 (format "hybrid"/"e4m3")
  backward  dX = Q(dY) . Q(W)        dY   -> E5M2 ("hybrid") or E4M3
            dW = Q(dY)^T . Q(X)
            db = sum_rows(dY)        (fp32 accumulate)

Under the "mxfp8" recipe every operand is quantised in blocks of 32 along the axis its GEMM contracts (X and W along
the input features for the forward, dY and W along the output features for dgrad, dY and X along the tokens for wgrad),
each block with its own power-of-two scale byte; there is no amax pass and no scaling state.  "blockwise" is the same
with blocks of 128 for activations and gradients and of 128 x 128 for the weight (one scale serves W and W^T), the
scale being the per-tensor rule on the block's amax rounded down to a power of two; the same GEMM multiplies both.

Every GEMM is issued in the "NT" form the MFMA wants (both operands contiguous
along the contraction axis); the cast+transpose kernel supplies the transposed
FP8 copies, and the forward keeps only the 1-byte ``Q(X)^T`` for wgrad instead of
the 2-byte activation.  Quantised weights (and their transposes) are cached until
the parameter changes, so gradient-accumulation microbatches and evaluation
re-quantise nothing.
"""

from __future__ import annotations

import logging
from typing import Any

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import native
from .amp import state as _state
from .amp.fp8 import FP8Recipe

logger = logging.getLogger(__name__)
_warned: set[str] = set()

ROLE_X, ROLE_W, ROLE_Y = 0, 1, 2      # forward roles (Y is reserved: outputs stay bf16)
ROLE_G, ROLE_DX = 0, 1                # backward roles (dX reserved likewise)
T, R, C = native.SCALE_TENSOR, native.SCALE_ROW, native.SCALE_COL


def _warn_once(msg: str) -> None:
    if msg not in _warned:
        _warned.add(msg)
        logger.warning(msg)


class _WeightCache:
    """Quantised weight + transpose, valid while the Parameter is unchanged."""

    __slots__ = ("key", "wq", "wq_t", "s_inv", "s_inv_t", "amax", "kept")

    def __init__(self):
        self.key = None
        self.wq = self.wq_t = self.s_inv = self.s_inv_t = self.amax = None
        # set by an Fp8ParamSet: what its codes were made from (address, version, format, recipe kind, margin); while
        # that still describes the weight and the recipe, the codes are used as they are, whatever the scale has done
        # since (under delayed scaling the set quantises once per optimizer step, not once per microbatch)
        self.kept = None


def _weight_key(weight: torch.Tensor, fmt: int, how: tuple) -> tuple:
    """What cached codes of a weight depend on: its storage, its contents (version counter), the format and
    how the scale is found."""
    return (weight.data_ptr(), _state.tensor_version(weight), fmt, how)


def _kept_stamp(weight: torch.Tensor, pol) -> tuple:
    return (weight.data_ptr(), _state.tensor_version(weight), pol.fmt_fwd, pol.kind, pol.margin)


def _quantise_dynamic(x2d: torch.Tensor, fmt: int, margin: int, need_t: bool, need_rowmajor: bool = True,
                      recipe: FP8Recipe | None = None, parts: torch.Tensor | None = None, out_t: torch.Tensor | None = None):
    """Per-tensor current scaling: amax pass, scale, cast (+transpose) pass.  The amax pass is
    skipped when the caller has the partial maxima, or when the kernel that produced x2d left them
    with the recipe."""
    if parts is None and recipe is not None:
        parts = recipe.take_parts(x2d)
    q, q_t, amax, _, scale_inv = native.quantize_dynamic(x2d, fmt, margin, want_rowmajor=need_rowmajor or not need_t,
                                                        want_transposed=need_t, parts=parts, out_t=out_t)
    return q, q_t, scale_inv, amax


def _input_key(x2d: torch.Tensor, kind: str, fmt: int, margin: int):
    return (x2d.data_ptr(), _state.tensor_version(x2d), tuple(x2d.shape), x2d.dtype, x2d.device, kind, fmt, margin)


def _quantise_input_shared(recipe: FP8Recipe, x2d: torch.Tensor, fmt: int, margin: int, need_t: bool):
    """Per-tensor quantisation of a Linear's input, reused by the next Linear that is fed the
    very same tensor (gate and up of an MLP, q/k/v of an attention block).  The entry keeps
    the tensor alive, so its address cannot be handed to another tensor while it is cached;
    an in-place change bumps ``_version`` and misses."""
    if not recipe.share_inputs:
        return _quantise_dynamic(x2d, fmt, margin, need_t, recipe=recipe)[:3]
    key = _input_key(x2d, "tensor", fmt, margin)
    hit = recipe.shared_input
    if hit is not None and hit["key"] == key and (hit["q_t"] is not None or not need_t):
        return hit["q"], hit["q_t"], hit["s_inv"]
    q, q_t, s_inv, _ = _quantise_dynamic(x2d, fmt, margin, need_t, recipe=recipe)
    entry = {"key": key, "x": x2d, "q": q, "q_t": q_t, "s_inv": s_inv}
    if hit is not None and hit.get("x") is x2d:          # keep the record of the conversion that produced x2d
        entry["src_key"], entry["src"] = hit.get("src_key"), hit.get("src")
    recipe.shared_input = entry
    return q, q_t, s_inv


def _block_cast(pol, x2d: torch.Tensor, fmt: int, want_rowmajor: bool, want_transposed: bool, weight: bool = False):
    """Codes and E8M0 scale bytes of the two block-scaled recipes: 32-element blocks (mxfp8) or 128-element blocks with
    128 x 128 ones for a weight (blockwise)."""
    if pol.kind == "mxfp8":
        return native.mx_cast(x2d, fmt, want_rowmajor=want_rowmajor, want_transposed=want_transposed,
                              scale_rule=pol.mx_scale_rule)
    return native.block_cast(x2d, fmt, pol.margin, two_d=weight, want_rowmajor=want_rowmajor, want_transposed=want_transposed)


def _mx_input_shared(recipe: FP8Recipe, x2d: torch.Tensor, fmt: int, need_t: bool):
    """Block-scaled codes and scale bytes of a Linear's input (blocks along the features; with need_t also of its
    transpose, blocks along the tokens), made once for the Linears fed by the very same tensor."""
    pol = recipe.recipe
    key = _input_key(x2d, (pol.kind, pol.mx_scale_rule), fmt, pol.margin)
    hit = recipe.shared_input if recipe.share_inputs else None
    if hit is not None and hit["key"] == key and (hit["q_t"] is not None or not need_t):
        return hit["q"], hit["s_inv"], hit["q_t"], hit["s_t"]
    q, sc, q_t, sc_t = _block_cast(pol, x2d, fmt, True, need_t)
    if recipe.share_inputs:
        entry = {"key": key, "x": x2d, "q": q, "q_t": q_t, "s_inv": sc, "s_t": sc_t}
        prev = recipe.shared_input
        if prev is not None and prev.get("x") is x2d:
            entry["src_key"], entry["src"] = prev.get("src_key"), prev.get("src")
        recipe.shared_input = entry
    return q, sc, q_t, sc_t


def _rowwise_input_shared(recipe: FP8Recipe, x2d: torch.Tensor, fmt: int, margin: int, need_t: bool):
    """Rowwise codes of a Linear's input: per-row scales for the forward GEMM and, with need_t, the transposed codes with
    per-column scales for wgrad, made once for the Linears fed by the very same tensor (two passes over x for q / k / v
    together instead of two each).  -> (xq, sx_inv, xq_t or None, sx_inv_t or None)."""
    key = _input_key(x2d, "rowwise", fmt, margin)
    hit = recipe.shared_input if recipe.share_inputs else None
    if hit is not None and hit["key"] == key and (hit["q_t"] is not None or not need_t):
        return hit["q"], hit["s_inv"], hit["q_t"], hit["s_t"]
    if need_t:
        q, s_inv, q_t, s_t, _, _ = native.quantize_rowcol(x2d, fmt, margin)
    else:
        (q, s_inv), q_t, s_t = _quantise_axis(x2d, fmt, margin, R, False), None, None
    if recipe.share_inputs:
        entry = {"key": key, "x": x2d, "q": q, "q_t": q_t, "s_inv": s_inv, "s_t": s_t}
        prev = recipe.shared_input
        if prev is not None and prev.get("x") is x2d:
            entry["src_key"], entry["src"] = prev.get("src_key"), prev.get("src")
        recipe.shared_input = entry
    return q, s_inv, q_t, s_t


def _converted_input(recipe: FP8Recipe, x2d: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """x2d in the compute dtype, contiguous.  Linears fed by the same tensor get the same
    converted tensor back (one conversion, and one quantisation downstream); autograd sees an
    ordinary tensor used twice."""
    key = (x2d.data_ptr(), _state.tensor_version(x2d), tuple(x2d.shape), tuple(x2d.stride()), x2d.dtype, x2d.device, dtype,
           torch.is_grad_enabled() and x2d.requires_grad)
    hit = recipe.shared_input
    if recipe.share_inputs and hit is not None and hit.get("src_key") == key:
        return hit["x"]
    out = x2d.to(dtype).contiguous()
    if recipe.share_inputs:
        recipe.shared_input = {"src_key": key, "src": x2d, "x": out, "key": None, "q": None, "q_t": None, "s_inv": None}
    return out


def _quantise_delayed(x2d: torch.Tensor, fmt: int, meta: "_state.ScalingMeta | None", role: int, need_t: bool,
                      need_rowmajor: bool = True, recipe: FP8Recipe | None = None, record: bool = True, margin: int = 0,
                      out_t: torch.Tensor | None = None):
    """Delayed scaling: one pass with the scale from the history, this step's partial maxima recorded with the role.
    record=False (a module in eval mode): the scales that training arrived at are used as they are and
    the histories are left alone; roles that do not exist yet (meta None) or have never been through a
    refresh still stand at the initial scale 1 (a weight of std 0.02 would land in the subnormals), so
    such a tensor is scaled from its own amax instead."""
    if not record and (meta is None or not meta.trained):
        q, q_t, scale_inv, _ = _quantise_dynamic(x2d, fmt, margin, need_t, need_rowmajor, out_t=out_t)
        return q, q_t, scale_inv
    slot = meta.amax_slot(role) if record else None
    if record:
        meta.note_record(recipe._store)
    # the scale is refreshed in place after the step; the cast hands back the inverse of the one it used
    return native.cast_delayed(x2d, meta.scale_of(role), fmt, amax_parts=slot, want_rowmajor=need_rowmajor or not need_t,
                               want_transposed=need_t, out_t=out_t)


def _quantise_axis(x2d: torch.Tensor, fmt: int, margin: int, mode: int, transposed: bool):
    """Rowwise recipe: one scale per row (mode R) or per column (mode C) of x2d.
    Returns the codes (transposed when asked) and the inverse scale vector."""
    amax = native.amax(x2d, mode)
    scale, scale_inv = native.scale_from_amax(amax, fmt, margin)
    if transposed:
        _, q = native.cast_transpose(x2d, scale, fmt, mode, want_rowmajor=False)
    else:
        q = native.cast(x2d, scale, fmt, mode)
    return q, scale_inv


class _Fp8LinearFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x2d: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None, module: "FP8Linear",
                recipe: FP8Recipe, out_dtype: torch.dtype):
        pol = recipe.recipe
        need_dgrad, need_wgrad = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        bias_f32 = None if bias is None else bias.detach().float()
        saved: dict[str, Any] = {}
        ctx.wgrad_direct = False

        if pol.kind in ("mxfp8", "blockwise"):
            fp8_wgrad = need_wgrad and recipe.wgrad
            xq, xs, xq_t, xs_t = _mx_input_shared(recipe, x2d, pol.fmt_fwd, fp8_wgrad)
            wq, ws, wq_t, ws_t = module._mx_weight(weight, recipe, need_t=need_dgrad)
            y = native.mx_gemm_nt(xq, xs, wq, ws, pol.fmt_fwd, pol.fmt_fwd, bias=bias_f32, out_dtype=out_dtype)
            if fp8_wgrad:
                saved["xq_t"], saved["xs_t"] = xq_t, xs_t
            if need_dgrad:
                saved["wq_t"], saved["ws_t"] = wq_t, ws_t
        elif pol.kind == "rowwise":
            # both operands of x in two passes over it: rows for this GEMM, columns (transposed) for wgrad; shared by the
            # Linears fed the very same tensor
            fp8_wgrad = need_wgrad and recipe.wgrad
            xq, sx_inv, xq_t, sx_inv_t = _rowwise_input_shared(recipe, x2d, pol.fmt_fwd, pol.margin, fp8_wgrad)
            if fp8_wgrad:
                saved["xq_t"], saved["sx_inv_t"] = xq_t, sx_inv_t
            if not recipe.cache_weights:
                module._wcache_rowwise.clear()          # the backward of this call still finds what is made now
            wq, sw_inv = module._rowwise_weight(weight, pol, "row", both=need_dgrad)
            y = native.gemm_nt(xq, wq, pol.fmt_fwd, pol.fmt_fwd, sx_inv, sw_inv, bias=bias_f32, out_dtype=out_dtype)
        else:
            # With whole 256 x 256 tiles wgrad reads the ROW-MAJOR codes of dy with the tokens as the slow
            # axis (native.gemm_layouts): dy, the largest tensor of the backward, gets no transposed copy.
            # x and w keep theirs: they are cold by the time the backward runs, and reading a cold operand
            # K-slow costs the GEMM more than the copy (measured), while dy has just been written.
            tokens, n_in, n_out = x2d.shape[0], x2d.shape[1], weight.shape[0]
            fp8_wgrad = need_wgrad and recipe.wgrad
            # (not when weight gradients are added into .grad by the GEMM: the kernel that reads dy as stored cannot
            # accumulate, and the detour through a workspace costs what the fusion saves: measured 500 us against
            # 475 us unfused for a 14336 x 4096 fp32 gradient, where the transposed route with the flag takes 395)
            ctx.wgrad_direct = (fp8_wgrad and recipe.direct_layouts and not recipe.fuse_wgrad_accumulation
                                and native.gemm_layouts_supported(n_out, n_in, tokens, weight.dtype)
                                and native.wgrad_direct_pays(n_out, n_in, tokens))
            if pol.kind == "delayed":
                # the histories see a forward only when it is part of training: the module in training mode AND
                # grad mode on (the reference's backend refreshes its state on the same condition), so a validation
                # pass under torch.no_grad() without model.eval() reads the scales and leaves the histories alone
                record = module._records()
                meta = module._meta(recipe, x2d.device, "fwd", create=record)
                xq, xq_t, sx_inv = _quantise_delayed(x2d, pol.fmt_fwd, meta, ROLE_X, fp8_wgrad, recipe=recipe,
                                                     record=record, margin=pol.margin)
            else:
                xq, xq_t, sx_inv = _quantise_input_shared(recipe, x2d, pol.fmt_fwd, pol.margin, fp8_wgrad)
            wq, wq_t, sw_inv = module._tensor_weight(weight, recipe, need_t=need_dgrad)
            y = native.gemm_nt(xq, wq, pol.fmt_fwd, pol.fmt_fwd, sx_inv, sw_inv, bias=bias_f32, out_dtype=out_dtype)
            if fp8_wgrad:
                saved["xq_t"], saved["sx_inv_t"] = xq_t, sx_inv
            if need_dgrad:
                saved["wq_t"], saved["sw_inv_t"] = wq_t, sw_inv
        if need_wgrad and not recipe.wgrad:
            saved["x_hp"] = x2d                      # wgrad=False: weight gradient in the activation dtype
        if pol.kind == "rowwise" and need_dgrad:
            saved["weight"] = weight                 # dgrad scales W per input channel, from the weight itself
        # Everything the backward reads goes through autograd's saved-tensor machinery: activation
        # checkpointing drops it after the forward and recomputes it, saved-tensor hooks (offloading) see it,
        # an in-place change of an input between forward and backward is detected, and the tensors are
        # released as soon as this node has run.
        ctx.saved_names = tuple(saved)
        ctx.save_for_backward(*saved.values())
        ctx.module, ctx.recipe = module, recipe
        ctx.need_wgrad, ctx.need_dgrad, ctx.has_bias = need_wgrad, need_dgrad, bias is not None
        ctx.x_dtype, ctx.w_dtype = x2d.dtype, weight.dtype
        ctx.bias_dtype = None if bias is None else bias.dtype
        return y

    @staticmethod
    def backward(ctx, dy: torch.Tensor):
        module, recipe = ctx.module, ctx.recipe
        saved = dict(zip(ctx.saved_names, ctx.saved_tensors))
        pol = recipe.recipe
        dy2d = dy if dy.is_contiguous() else dy.contiguous()
        if dy2d.dtype not in (torch.bfloat16, torch.float32):
            dy2d = dy2d.to(torch.bfloat16)
        dx = dw = db = None
        fp8_wgrad = ctx.need_wgrad and recipe.wgrad

        if pol.kind in ("mxfp8", "blockwise"):
            if ctx.need_dgrad or fp8_wgrad:
                # one pass over dy: blocks along the output features for dgrad, along the tokens (transposed) for wgrad
                gq, gs, gq_t, gs_t = _block_cast(pol, dy2d, pol.fmt_bwd, ctx.need_dgrad, fp8_wgrad)
            if ctx.need_dgrad:
                dx = native.mx_gemm_nt(gq, gs, saved["wq_t"], saved["ws_t"], pol.fmt_bwd, pol.fmt_fwd, out_dtype=ctx.x_dtype)
            if fp8_wgrad:
                dw = native.mx_gemm_nt(gq_t, gs_t, saved["xq_t"], saved["xs_t"], pol.fmt_bwd, pol.fmt_fwd, out_dtype=ctx.w_dtype)
        elif pol.kind == "rowwise":
            if ctx.need_dgrad and fp8_wgrad:
                gq, sg_inv, gq_t, sg_inv_t, _, _ = native.quantize_rowcol(dy2d, pol.fmt_bwd, pol.margin)
            elif ctx.need_dgrad:
                gq, sg_inv = _quantise_axis(dy2d, pol.fmt_bwd, pol.margin, R, False)
            elif fp8_wgrad:
                gq_t, sg_inv_t = _quantise_axis(dy2d, pol.fmt_bwd, pol.margin, C, True)
            if ctx.need_dgrad:
                wq_t, sw_inv_t = module._rowwise_weight(saved["weight"], pol, "col")
                dx_into = getattr(ctx, "dx_into", None)      # a later member of a sibling group adds into the group's dx
                if dx_into is not None:
                    dx = native.gemm_nt(gq, wq_t, pol.fmt_bwd, pol.fmt_fwd, sg_inv, sw_inv_t, out=dx_into, accumulate=True)
                else:
                    dx = native.gemm_nt(gq, wq_t, pol.fmt_bwd, pol.fmt_fwd, sg_inv, sw_inv_t, out_dtype=ctx.x_dtype)
            if fp8_wgrad:
                dw = native.gemm_nt(gq_t, saved["xq_t"], pol.fmt_bwd, pol.fmt_fwd, sg_inv_t, saved["sx_inv_t"],
                                    out_dtype=ctx.w_dtype)
        else:
            # the transposed codes of dy are only needed by a wgrad that cannot read the row-major ones
            g_t_needed = fp8_wgrad and not ctx.wgrad_direct
            g_rm_needed = ctx.need_dgrad or (fp8_wgrad and ctx.wgrad_direct)
            # a member of a group whose weight gradients are computed by ONE GEMM: its transposed codes go into the
            # group's buffer and the GEMM is left to the group (_Fp8LinearGroupFn.backward)
            joint = getattr(ctx, "wgrad_joint", None)
            gq_t_out = joint["codes_t"] if joint is not None else None
            if ctx.need_dgrad or fp8_wgrad:
                if pol.kind == "delayed":
                    meta = module._meta(recipe, dy2d.device, "bwd", create=module.training)
                    gq, gq_t, sg_inv = _quantise_delayed(dy2d, pol.fmt_bwd, meta, ROLE_G, g_t_needed, g_rm_needed,
                                                         recipe=recipe, record=module.training, margin=pol.margin, out_t=gq_t_out)
                else:
                    parts = recipe.take_parts(dy2d)
                    if ctx.has_bias and native.colsum_supported(dy2d):
                        # the amax pass also adds up the columns: the bias gradient costs no extra read of dy.  It
                        # runs for the column sums even when the producer of dy left its partial maxima (which are
                        # the same numbers): one pass of this kernel is cheaper than a separate sum over the rows
                        parts, colsum = native.amax_parts_colsum(dy2d)
                        db = colsum.to(ctx.bias_dtype)
                    gq, gq_t, sg_inv, _ = _quantise_dynamic(dy2d, pol.fmt_bwd, pol.margin, g_t_needed, g_rm_needed,
                                                            parts=parts, out_t=gq_t_out)
            if ctx.need_dgrad:
                # a member of a group of Linears fed by one tensor leaves its operands to the group's one GEMM over
                # all members, or adds its share into the group's gradient (the GEMM's accumulate flag), instead of
                # leaving the sum to a separate pass
                dx_pairs = getattr(ctx, "dx_pairs", None)
                dx_into = getattr(ctx, "dx_into", None)
                if dx_pairs is not None:
                    dx_pairs.append((gq, saved["wq_t"], sg_inv, saved["sw_inv_t"]))
                elif dx_into is not None:
                    dx = native.gemm_nt(gq, saved["wq_t"], pol.fmt_bwd, pol.fmt_fwd, sg_inv, saved["sw_inv_t"],
                                        out=dx_into, accumulate=True)
                else:
                    dx = native.gemm_nt(gq, saved["wq_t"], pol.fmt_bwd, pol.fmt_fwd, sg_inv, saved["sw_inv_t"],
                                        out_dtype=ctx.x_dtype)
            if fp8_wgrad and joint is not None:
                joint["sg_inv"] = sg_inv             # the group multiplies: dW rows of this member = dY^T codes . X^T codes
            elif fp8_wgrad:
                # gradient accumulation over microbatches: with recipe.fuse_wgrad_accumulation the product is added
                # straight into the existing .grad (and autograd is handed nothing to add)
                grad_buf = module.weight.grad if recipe.fuse_wgrad_accumulation else None
                into = grad_buf is not None and grad_buf.dtype == ctx.w_dtype and grad_buf.is_contiguous() and grad_buf.is_cuda \
                    and tuple(grad_buf.shape) == (module.out_features, module.in_features)
                if ctx.wgrad_direct:        # dW = dY^T . X with dY [tokens, N] as stored, X^T from the forward
                    dw = native.gemm_layouts(gq, saved["xq_t"], pol.fmt_bwd, pol.fmt_fwd, native.K_SLOW, native.K_FAST,
                                             sg_inv, saved["sx_inv_t"], out=grad_buf if into else None,
                                             out_dtype=ctx.w_dtype, accumulate=into)
                else:
                    dw = native.gemm_nt(gq_t, saved["xq_t"], pol.fmt_bwd, pol.fmt_fwd, sg_inv, saved["sx_inv_t"],
                                        out=grad_buf if into else None, out_dtype=ctx.w_dtype, accumulate=into)
                if into:
                    dw = None
        if ctx.need_wgrad and not recipe.wgrad:
            dw = (dy2d.t().to(saved["x_hp"].dtype) @ saved["x_hp"]).to(ctx.w_dtype)
        if ctx.has_bias and db is None:
            if dy2d.is_cuda and native.colsum_supported(dy2d):
                # delayed and rowwise scaling have no amax pass to ride on: the same kernel, for its column sums only
                db = native.amax_parts_colsum(dy2d)[1].to(ctx.bias_dtype)
            else:
                db = dy2d.sum(dim=0, dtype=torch.float32).to(ctx.bias_dtype)
        return dx, dw, db, None, None, None


class _MemberCtx:
    """What ``_Fp8LinearFn.forward`` / ``backward`` expect of an autograd context, for one member of a group: the tensors
    it saves are collected by the group's own context (so they still go through autograd's saved-tensor machinery)."""

    def __init__(self, needs_input_grad: tuple):
        self.needs_input_grad = needs_input_grad
        self.saved_tensors: tuple = ()

    def save_for_backward(self, *tensors: torch.Tensor) -> None:
        self.saved_tensors = tensors


class _Fp8LinearGroupFn(torch.autograd.Function):
    """Several FP8 Linears applied to ONE input (q/k/v of an attention block, gate/up of a gated MLP) as one autograd
    node: forward = the members' forwards (they share the quantised input anyway), backward = the members' backwards
    with the data gradients summed by the GEMMs themselves: ONE GEMM whose contraction runs through all members'
    operands where the shapes allow (``native.gemm_nt_sum``), else the first member writes dx and every further one adds
    its product into it (``accumulate``); separate nodes leave two extra passes over dx per block to autograd."""

    @staticmethod
    def forward(ctx, x2d: torch.Tensor, recipe: FP8Recipe, out_dtype: torch.dtype, modules: tuple, *params: torch.Tensor | None):
        ctx.set_materialize_grads(False)         # an output that did not reach the loss arrives as None, not as zeros
        subs, outs, saved, spans = [], [], [], []
        for i, mod in enumerate(modules):
            weight, bias = params[2 * i], params[2 * i + 1]
            sub = _MemberCtx((ctx.needs_input_grad[0], ctx.needs_input_grad[4 + 2 * i], ctx.needs_input_grad[5 + 2 * i],
                              False, False, False))
            outs.append(_Fp8LinearFn.forward(sub, x2d, weight, bias, mod, recipe, out_dtype))
            spans.append((len(saved), len(sub.saved_tensors)))
            saved.extend(sub.saved_tensors)
            sub.saved_tensors = ()
            subs.append(sub)
        ctx.save_for_backward(*saved)
        ctx.subs, ctx.spans = subs, spans
        return tuple(outs)

    @staticmethod
    def _joint_wgrad(ctx, tensors, dys):
        """The members whose weight gradients one GEMM computes: those that would each run a GEMM of few 128 x 128 tiles
        over a transposed copy of their dy (``native.wgrad_direct_pays`` false: k and v of a grouped-query attention
        block, 1024 x 4096 each) and contract the same codes of X^T.  Their transposed dy codes are written side by side
        into one buffer, the scales become a per-row vector, and dW comes out as one [sum N, K] matrix whose row ranges
        are the members' gradients: twice the tiles per launch fill the chip where each alone leaves every compute unit
        with one block (measured, 8192 tokens: 2 x [1024 x 4096] 83.0 us, one [2048 x 4096] 65.2 us).
        -> (indices, codes_t buffer, X^T codes, its inverse scale) or None."""
        recipe = ctx.subs[0].recipe
        if not getattr(recipe, "fuse_sibling_wgrad", True) or recipe.fuse_wgrad_accumulation or not recipe.wgrad:
            return None
        if recipe.recipe.kind not in ("tensorwise", "delayed"):
            return None
        picked, xq_t, sx_inv_t, w_dtype = [], None, None, None
        for i, (sub, (first, count), dy) in enumerate(zip(ctx.subs, ctx.spans, dys)):
            if dy is None or not sub.need_wgrad or sub.wgrad_direct or "xq_t" not in sub.saved_names:
                continue
            saved = dict(zip(sub.saved_names, tensors[first:first + count]))
            if xq_t is None:
                xq_t, sx_inv_t, w_dtype = saved["xq_t"], saved["sx_inv_t"], sub.w_dtype
            elif saved["xq_t"].data_ptr() != xq_t.data_ptr() or saved["sx_inv_t"].data_ptr() != sx_inv_t.data_ptr() or sub.w_dtype != w_dtype:
                continue
            picked.append(i)
        if len(picked) < 2:
            return None
        tokens = xq_t.shape[1]
        rows = sum(ctx.subs[i].module.out_features for i in picked)
        return picked, torch.empty((rows, tokens), dtype=torch.uint8, device=xq_t.device), xq_t, sx_inv_t

    @staticmethod
    def _dgrad_in_one_gemm(ctx, dys) -> "list | None":
        """An empty list for the members to put their dgrad operands in (codes of dy, codes of W^T, the two inverse
        scales) where ONE GEMM computes dx = sum over members of dy_s . W_s (``native.gemm_nt_sum``), else None: the
        members then add into dx one by one.  One launch where per-tensor scales and the shapes allow: the k and v
        shares of a grouped-query block (contractions of 1024) are, added into a cold 64 MB dx, bound by reading and
        writing it (63 us each at 8192 tokens against 40 for the bare product); carried through one set of
        accumulators they cost what their share of the contraction costs."""
        recipe = ctx.subs[0].recipe
        if not getattr(recipe, "fuse_dgrad_gemm", True) or recipe.recipe.kind not in ("tensorwise", "delayed"):
            return None
        live = [sub for sub, dy in zip(ctx.subs, dys) if dy is not None and sub.need_dgrad]
        if len(live) < 2 or any(dy is not None and not sub.need_dgrad for sub, dy in zip(ctx.subs, dys)):
            return None
        tokens = next(dy for dy in dys if dy is not None).shape[0]
        if not native.dgrad_sum_in_one_launch(tokens, live[0].module.in_features, [sub.module.out_features for sub in live]):
            return None
        return []

    @staticmethod
    def backward(ctx, *dys: torch.Tensor | None):
        tensors = ctx.saved_tensors
        dx = None
        grads: list = []
        joint = _Fp8LinearGroupFn._joint_wgrad(ctx, tensors, dys)
        if joint is not None:
            at = 0
            for i in joint[0]:
                n = ctx.subs[i].module.out_features
                ctx.subs[i].wgrad_joint = {"codes_t": joint[1][at:at + n], "rows": (at, at + n)}
                at += n
        dx_pairs = _Fp8LinearGroupFn._dgrad_in_one_gemm(ctx, dys)
        for sub, (first, count), dy in zip(ctx.subs, ctx.spans, dys):
            if dy is None:                       # this member's output did not reach the loss
                grads += [None, None]
                continue
            sub.saved_tensors = tensors[first:first + count]
            sub.dx_pairs = dx_pairs
            sub.dx_into = dx if (dx is not None and sub.need_dgrad) else None
            dxi, dw, db, _, _, _ = _Fp8LinearFn.backward(sub, dy)
            sub.saved_tensors = ()
            sub.dx_pairs = None
            if dxi is not None and dx is None:
                dx = dxi
            grads += [dw, db]
        if dx_pairs:
            pol = ctx.subs[0].recipe.recipe
            gqs, wq_ts, sg_invs, sw_invs = zip(*dx_pairs)
            dx = native.gemm_nt_sum(list(gqs), list(wq_ts), pol.fmt_bwd, pol.fmt_fwd, list(sg_invs), list(sw_invs),
                                    out_dtype=ctx.subs[0].x_dtype)
        if joint is not None:
            picked, codes_t, xq_t, sx_inv_t = joint
            pol = ctx.subs[0].recipe.recipe
            parts = [ctx.subs[i].wgrad_joint for i in picked]
            sa = torch.cat([p["sg_inv"].expand(p["rows"][1] - p["rows"][0]) for p in parts])
            dw_all = native.gemm_nt(codes_t, xq_t, pol.fmt_bwd, pol.fmt_fwd, sa, sx_inv_t, out_dtype=ctx.subs[picked[0]].w_dtype)
            for i, p in zip(picked, parts):
                grads[2 * i] = dw_all[p["rows"][0]:p["rows"][1]]
                ctx.subs[i].wgrad_joint = None
        return (dx, None, None, None, *grads)


@torch.compiler.disable
def linear_group(x: torch.Tensor, modules: "tuple[FP8Linear, ...]") -> tuple[torch.Tensor, ...] | None:
    """``tuple(m(x) for m in modules)`` as one autograd node (see ``_Fp8LinearGroupFn``), or None where the members
    cannot run that way (no recipe, a block-scaled recipe, shapes the FP8 path refuses): the caller
    then applies the modules one by one."""
    recipe = _state.active_recipe()
    if recipe is None or recipe.recipe.kind not in ("tensorwise", "delayed", "rowwise") or not recipe.fuse_dgrad_sum:
        return None
    if not all(m._fp8_eligible(x) for m in modules):
        return None
    compute_dtype = torch.get_autocast_dtype("cuda") if torch.is_autocast_enabled("cuda") else x.dtype
    if compute_dtype not in (torch.bfloat16, torch.float32):
        compute_dtype = torch.bfloat16
    k = modules[0].in_features
    x2d = x.reshape(-1, k)
    if x2d.dtype != compute_dtype or not x2d.is_contiguous():
        x2d = _converted_input(recipe, x2d, compute_dtype)
    params: list = []
    for m in modules:
        m.fp8_calls += 1
        m._note_grad_mode()
        params += [m.weight, m.bias]
    outs = _Fp8LinearGroupFn.apply(x2d, recipe, compute_dtype, tuple(modules), *params)
    return tuple(y.reshape(*x.shape[:-1], m.out_features) for y, m in zip(outs, modules))


class SiblingGroup:
    """Linears of one parent module that are fed the same tensor in its forward (``wq``, ``wk``, ``wv`` of the
    reference's attention block, attention.py:317-319; ``w1``, ``w2`` of its gated MLP, mlp.py:76-78).  The parent's
    forward is not touched: the member that is called first computes the outputs of ALL members through
    ``linear_group`` and keeps the others' until they are asked for with the very same tensor (same address, version,
    shape and strides).  A member called with another tensor simply runs on its own; after that has happened the group stands
    down for good (its members are evidently not fed one tensor: cross-attention, say), so that nothing is computed
    for nothing twice."""

    def __init__(self, modules: "list[FP8Linear]"):
        self.modules = tuple(modules)
        self.pending: dict = {}
        self.key = None
        self.x = None
        self.misses = 0
        self.groups_run = 0              # forwards that ran as one node for all members (for tests / logging)
        for m in self.modules:
            m._siblings = self

    def clear(self) -> None:
        self.pending, self.key, self.x = {}, None, None

    @torch.compiler.disable          # like FP8Linear._forward_fp8: runs as written, between the compiled parts of a model
    def forward(self, member: "FP8Linear", x: torch.Tensor) -> torch.Tensor:
        # the same values at the same address: the same tensor object, or another handle on it (a graph compiler hands
        # the pieces of a model it runs separately fresh handles on the same storage)
        key = (x.data_ptr(), _state.tensor_version(x), tuple(x.shape), tuple(x.stride()), x.dtype, x.requires_grad)
        if self.key == key and id(member) in self.pending:
            out = self.pending.pop(id(member))
            if not self.pending:
                self.clear()
            return out
        if self.pending:                 # outputs made for siblings that were then fed something else
            self.misses += 1
            self.clear()
        if self.misses or not torch.is_grad_enabled() or not x.requires_grad:
            return member._forward_fp8(x)
        outs = linear_group(x, self.modules)
        if outs is None:
            return member._forward_fp8(x)
        recipe = _state.active_recipe()
        recipe._sibling_groups.add(self)
        self.groups_run += 1
        self.key, self.x = key, x        # the entry keeps x alive: its address cannot be handed to another tensor meanwhile
        self.pending = {id(m): y for m, y in zip(self.modules, outs) if m is not member}
        return outs[self.modules.index(member)]


def keep_layers_in_bf16(model: nn.Module, at_start: int = 1, at_end: int = 1) -> list[str]:
    """``first_last_layers_bf16`` with ``num_layers_at_start_in_bf16`` / ``num_layers_at_end_in_bf16``
    (optimus_dl/modules/optim/config.py:44-49,62-66: "retain first and last N layers in BF16"; the reference declares
    the keys and never reads them).  The layers are the entries of the model's block list: the ``nn.ModuleList`` with
    the most entries among those whose every entry holds an FP8 Linear (``transformer.h`` of the reference's GPT-2 /
    Llama / Qwen3 trees).  The FP8 Linears inside its first ``at_start`` and last ``at_end`` entries get
    ``fp8_enabled = False`` and run in the autocast dtype; everything else (embedding, head, the other blocks) is left as
    it is.  Returns the qualified names of the Linears switched off (empty when no such list exists)."""
    best_name, best = "", None
    for name, mod in model.named_modules():
        if isinstance(mod, nn.ModuleList) and len(mod) > 0 and (best is None or len(mod) > len(best)):
            if all(any(isinstance(m, FP8Linear) for m in entry.modules()) for entry in mod):
                best_name, best = name, mod
    if best is None:
        return []
    n = len(best)
    picked = sorted(set(range(min(max(at_start, 0), n))) | set(range(max(n - max(at_end, 0), 0), n)))
    names = []
    for i in picked:
        for sub, m in best[i].named_modules():
            if isinstance(m, FP8Linear):
                m.fp8_enabled = False
                names.append(".".join(x for x in (best_name, str(i), sub) if x))
    return names


class FP8Linear(nn.Linear):
    """Drop-in ``nn.Linear`` with an FP8 fast path (see the module docstring)."""

    _siblings: "SiblingGroup | None" = None      # set on the instance by a SiblingGroup that this Linear is a member of
    # False: this Linear stays in the autocast dtype under an FP8 recipe too (``first_last_layers_bf16`` of the
    # reference's config, optimus_dl/modules/optim/config.py:62-66; set by ``keep_layers_in_bf16``)
    fp8_enabled: bool = True

    def __init__(self, in_features: int, out_features: int, bias: bool = True, device=None, dtype=None, **kwargs: Any):
        super().__init__(in_features, out_features, bias=bias, device=device, dtype=dtype)
        self.use_bias = bias
        self.kwargs = dict(kwargs)           # backend-specific options (e.g. sequence_parallel): accepted, unused on one GPU
        self._init_fp8_state()

    def _init_fp8_state(self) -> None:
        self._wcache = _WeightCache()
        self._wcache_rowwise: dict[str, tuple] = {}
        self._metas: dict[tuple, "_state.ScalingMeta"] = {}
        self.fp8_meta: dict[str, "_state.ScalingMeta"] = {}
        self.fp8_calls = 0                   # forwards that actually took the FP8 path (for tests / logging)

    # Quantised weights and scaling-state views are per-process run-time state: a copy or a pickle of the module
    # starts without them (they are rebuilt on first use) instead of dragging device buffers and arenas along.
    _RUNTIME_STATE = ("_wcache", "_wcache_rowwise", "_metas", "fp8_meta", "fp8_calls", "_siblings", "_grad_mode")

    def __getstate__(self) -> dict:
        state = self.__dict__.copy()
        for name in self._RUNTIME_STATE:
            state.pop(name, None)
        return state

    def __setstate__(self, state: dict) -> None:
        super().__setstate__(state)
        self._init_fp8_state()

    @classmethod
    def from_linear(cls, linear: nn.Linear, **kwargs: Any) -> "FP8Linear":
        """Re-wrap an existing layer, SHARING its Parameter objects."""
        new = cls.__new__(cls)
        nn.Module.__init__(new)
        new.in_features, new.out_features = linear.in_features, linear.out_features
        new.weight = linear.weight
        if linear.bias is not None:
            new.bias = linear.bias
        else:
            new.register_parameter("bias", None)
        new.use_bias = linear.bias is not None
        new.kwargs = dict(kwargs)
        new.training = linear.training
        new._init_fp8_state()
        return new

    @property
    def _te_linear(self) -> "FP8Linear":
        """The reference nests the backend layer under this name; here it is the module itself."""
        return self

    # ------------------------------------------------------------ scaling state
    def _meta(self, recipe: FP8Recipe, device: torch.device, direction: str, create: bool = True) -> "_state.ScalingMeta | None":
        """This module's delayed-scaling roles for one direction.  Keyed by what the state depends on
        (history length, formats, device), not by the recipe object: the reference's backend keeps
        ``fp8_meta`` on the layer, and a second recipe of the same shape -- the one an evaluation forward
        builds per call -- continues with the scales the first one measured.  create=False: None when
        the roles do not exist yet (nothing is reserved)."""
        pol = recipe.recipe
        key = (pol.amax_history_len, pol.fmt_fwd, pol.fmt_bwd, str(device), direction)
        meta = self._metas.get(key)
        if meta is None:
            if not create:
                return None
            fmts = [pol.fmt_fwd] * 3 if direction == "fwd" else [pol.fmt_bwd] * 2
            meta = recipe.reserve_meta(device, direction, fmts)
            self._metas[key] = meta
        self.fp8_meta["scaling_fwd" if direction == "fwd" else "scaling_bwd"] = meta
        return meta

    def _records(self) -> bool:
        """Whether the forward in progress feeds the delayed-scaling histories: training mode and grad mode, as noted
        by ``_note_grad_mode`` before the autograd function was entered (inside it grad mode is always off)."""
        return self.training and self.__dict__.get("_grad_mode", True)

    def _note_grad_mode(self) -> None:
        self.__dict__["_grad_mode"] = torch.is_grad_enabled()

    def _tensor_weight(self, weight: torch.Tensor, recipe: FP8Recipe, need_t: bool):
        """Per-tensor quantised weight (and transpose), cached on the parameter version."""
        pol = recipe.recipe
        c = self._wcache
        if c.kept is not None and recipe.cache_weights and c.kept == _kept_stamp(weight, pol):
            return c.wq, c.wq_t, c.s_inv
        record = self._records()
        meta = None
        # the codes depend on the parameter's contents, the format and how the scale is found; under delayed
        # scaling also on the scale in force, which changes with every refresh of the arena
        if pol.kind == "delayed":
            meta = self._meta(recipe, weight.device, "fwd", create=record)
            how = ("delayed", pol.amax_history_len, id(meta.arena), meta.arena.epoch, record) if meta is not None else ("own amax", pol.margin)
        else:
            how = (pol.kind, pol.margin)
        key = _weight_key(weight, pol.fmt_fwd, how)
        fresh = c.key != key or not recipe.cache_weights
        if fresh or (need_t and c.wq_t is None):
            w2d = weight.detach()
            if pol.kind == "delayed":
                c.wq, c.wq_t, c.s_inv = _quantise_delayed(w2d, pol.fmt_fwd, meta, ROLE_W, need_t, recipe=recipe, record=record,
                                                          margin=pol.margin)
                c.amax = meta.amax_slot(ROLE_W).clone() if record else None     # only this weight ever writes that slot
            else:
                c.wq, c.wq_t, c.s_inv, c.amax = _quantise_dynamic(w2d, pol.fmt_fwd, pol.margin, need_t)
            c.key = key
        elif pol.kind == "delayed" and record:
            # cached codes are reused; this step's history still has to see the weight's amax
            slot = meta.amax_slot(ROLE_W)
            torch.maximum(slot, c.amax, out=slot)
            meta.note_record(recipe._store)
        return c.wq, c.wq_t, c.s_inv

    def _rowwise_weight(self, weight: torch.Tensor, pol, axis: str, both: bool = False):
        """Rowwise recipe: W scaled per output channel (fwd) or per input channel, transposed (dgrad).
        both: the other one will be asked for too (a backward follows): make them in one go."""
        key = _weight_key(weight, pol.fmt_fwd, ("rowwise", pol.margin))
        hit = self._wcache_rowwise.get(axis)
        if hit is not None and hit[0] == key:
            return hit[1], hit[2]
        w2d = weight.detach()
        if both:
            q, s_inv, q_t, s_inv_t, _, _ = native.quantize_rowcol(w2d, pol.fmt_fwd, pol.margin)
            self._wcache_rowwise["row"] = (key, q, s_inv)
            self._wcache_rowwise["col"] = (key, q_t, s_inv_t)
            return self._wcache_rowwise[axis][1], self._wcache_rowwise[axis][2]
        if axis == "row":
            q, s_inv = _quantise_axis(w2d, pol.fmt_fwd, pol.margin, R, False)
        else:
            q, s_inv = _quantise_axis(w2d, pol.fmt_fwd, pol.margin, C, True)
        self._wcache_rowwise[axis] = (key, q, s_inv)
        return q, s_inv

    def _mx_weight(self, weight: torch.Tensor, recipe: FP8Recipe, need_t: bool):
        """Block-scaled codes and scale bytes of W (blocks along the input features) and, with need_t, of W^T (blocks along
        the output features, for dgrad; under the blockwise recipe both share the scales of the 128 x 128 blocks); kept
        while the Parameter is unchanged."""
        pol = recipe.recipe
        fmt = pol.fmt_fwd
        key = _weight_key(weight, fmt, (pol.kind, pol.margin, pol.mx_scale_rule))
        hit = self._wcache_rowwise.get("mx")
        if hit is not None and hit[0] == key and recipe.cache_weights and (hit[3] is not None or not need_t):
            return hit[1:]
        q, sc, q_t, sc_t = _block_cast(pol, weight.detach(), fmt, True, need_t, weight=True)
        self._wcache_rowwise["mx"] = (key, q, sc, q_t, sc_t)
        return q, sc, q_t, sc_t

    # ------------------------------------------------------------------ forward
    def _fp8_eligible(self, x: torch.Tensor) -> bool:
        if not self.fp8_enabled or not x.is_cuda or not self.weight.is_cuda:
            return False
        if self.weight.dtype not in (torch.bfloat16, torch.float32):
            _warn_once(f"FP8Linear: weight dtype {self.weight.dtype} is not bf16/fp32; running as a plain Linear")
            return False
        tokens = x.numel() // max(self.in_features, 1)
        recipe = _state.active_recipe()
        # MXFP8 blocks are 32 long along every axis a GEMM of this layer contracts (features in and out, tokens), the
        # blocks of the blockwise recipe 128
        kind = recipe.recipe.kind if recipe is not None else ""
        mult = 32 if kind == "mxfp8" else (128 if kind == "blockwise" else 16)
        if self.in_features % mult or self.out_features % mult or tokens % mult or tokens == 0:
            _warn_once(
                f"FP8Linear({self.in_features}->{self.out_features}) with {tokens} tokens: sizes must be multiples "
                f"of {mult} for the FP8 kernels; this call runs as a plain Linear"
            )
            return False
        return True

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if _state.active_recipe() is None or not self.fp8_enabled:
            return F.linear(x, self.weight, self.bias)
        siblings = self._siblings
        if siblings is not None:
            return siblings.forward(self, x)
        return self._forward_fp8(x)

    # The FP8 path calls the native library through ctypes and keeps per-step state on the recipe: a graph
    # compiler (the reference has a torch.compile transform, model_transforms/compile.py) must not trace into
    # it.  Marked like this it runs as written, between the compiled parts of the model.
    @torch.compiler.disable
    def _forward_fp8(self, x: torch.Tensor) -> torch.Tensor:
        recipe = _state.active_recipe()
        if recipe is None or not self._fp8_eligible(x):
            return F.linear(x, self.weight, self.bias)
        if torch.is_autocast_enabled("cuda"):
            compute_dtype = torch.get_autocast_dtype("cuda")
        else:
            compute_dtype = x.dtype
        if compute_dtype not in (torch.bfloat16, torch.float32):
            compute_dtype = torch.bfloat16
        x2d = x.reshape(-1, self.in_features)
        if x2d.dtype != compute_dtype or not x2d.is_contiguous():
            x2d = _converted_input(recipe, x2d, compute_dtype)
        self.fp8_calls += 1
        self._note_grad_mode()
        y = _Fp8LinearFn.apply(x2d, self.weight, self.bias, self, recipe, compute_dtype)
        return y.reshape(*x.shape[:-1], self.out_features)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}, fp8=True"


class Fp8ParamSet:
    """The weights of a model's FP8 Linears kept quantised between optimizer steps (``fp8.param: true``,
    optimus_dl/modules/optim/config.py:36-37,56: declared there and never read).

    Without it every ``FP8Linear`` quantises its own weight on the first forward after the weight changed (under
    delayed scaling: in every forward, with the scale refreshed since): one or two launches per weight (a model of 196
    Linears: up to 392 launches and as many allocations per step).  With it, :meth:`sync` quantises all of them in TWO
    launches (current scaling) or ONE (delayed scaling) into buffers that live as long as the set, and stamps every
    module's weight cache, so the forwards that follow launch nothing for the weights.

    * tensorwise: codes and scales are the same bits as on the per-module route.
    * delayed: the weights are cast with the scales in force at the ``sync`` and their maxima recorded for the next
      refresh; the microbatches of one optimizer step all use these codes (what the reference's backend does when it is
      told that the weights are cached), where the per-module route casts again in every forward.  With one forward per
      optimizer step both routes give the same bits.

    ``sync`` belongs right after ``optimizer.step()`` (``attach`` registers it as a step post-hook when handed the
    optimizer); it rewrites the buffers in place, so no backward that still needs the previous codes may be pending,
    the same rule as for the optimizer's own in-place update.  A weight that changes without a ``sync`` (a checkpoint
    load, a manual edit) is simply quantised by its module on the next forward, as without the set.  The rowwise
    recipe keeps its per-module route."""

    def __init__(self, modules: list["FP8Linear"], recipe: FP8Recipe):
        pol = recipe.recipe
        if pol.kind not in ("tensorwise", "delayed"):
            raise ValueError(f"Fp8ParamSet serves the tensorwise and delayed recipes, not '{pol.kind}'")
        self.recipe = recipe
        self.modules: list[FP8Linear] = []
        self.skipped: list[FP8Linear] = []          # shapes / dtypes the multi-tensor route does not take: per-module route
        for m in modules:
            (self.modules if native.MultiTensorPlan.eligible(m.weight.detach()) else self.skipped).append(m)
        self._plan: native.MultiTensorPlan | None = None
        self._index: list[int] = []
        self._metas: list = []
        self.syncs = 0

    def _build(self) -> None:
        pol = self.recipe.recipe
        sources, index, seen, scales, parts, metas = [], [], {}, [], [], []
        for m in self.modules:
            w = m.weight.detach()
            at = seen.get(w.data_ptr())
            if at is None:                           # Linears that share one Parameter share its codes
                at = seen[w.data_ptr()] = len(sources)
                sources.append(w)
                if pol.kind == "delayed":            # the first module of a shared Parameter lends its weight role
                    meta = m._meta(self.recipe, w.device, "fwd")
                    scales.append(meta.scale_of(ROLE_W))
                    parts.append(meta.amax_slot(ROLE_W))
                    metas.append(meta)
            index.append(at)
        if not sources:
            self._plan = None
        elif pol.kind == "delayed":
            self._plan = native.MultiTensorPlan(sources, pol.fmt_fwd, pol.margin, scales=scales, parts=parts)
        else:
            self._plan = native.MultiTensorPlan(sources, pol.fmt_fwd, pol.margin)
        self._index, self._metas = index, metas
        # the rows of each arena's strip table that hold these weights' partial maxima
        rows: dict = {}
        for meta in metas:
            rows.setdefault(meta.arena, []).append(meta.first + ROLE_W)
        self._w_rows = {arena: torch.tensor(idx, dtype=torch.long, device=arena.parts.device) for arena, idx in rows.items()}
        self._w_snap: dict = {}

    @torch.no_grad()
    def sync(self) -> None:
        """Quantise every weight of the set now (on the current stream)."""
        if not self.modules:
            return
        if self._plan is None or len(self._index) != len(self.modules) or self._plan.stale() or \
                any(m.weight.data_ptr() != self._plan.sources[i].data_ptr() for m, i in zip(self.modules, self._index)):
            self._build()                            # first use, or a parameter's storage moved (.to(), a new optimizer state)
        plan, pol = self._plan, self.recipe.recipe
        plan.run()
        for meta in self._metas:                     # delayed: the next refresh has to fold what was just recorded
            meta.note_record(self.recipe._store)
        # ... and so has every later refresh until the next sync: the strips are cleared by each refresh (one per
        # microbatch), while the kept codes launch nothing that would record the weights' maxima again
        self._w_snap = {arena: arena.parts.index_select(0, idx) for arena, idx in self._w_rows.items()}
        how = (pol.kind, pol.margin)
        for m, i in zip(self.modules, self._index):
            c = m._wcache
            c.wq, c.wq_t, c.s_inv = plan.codes[i], plan.codes_t[i], plan.dyn[i, 2:3]
            c.kept = _kept_stamp(m.weight, pol)
            if pol.kind == "tensorwise":
                c.amax = plan.dyn[i, 0:1]
                c.key = _weight_key(m.weight, pol.fmt_fwd, how)
            else:
                c.amax, c.key = None, None
        self.syncs += 1

    def refold(self, arena) -> None:
        """Called by the recipe before it refreshes ``arena``: the maxima recorded at the last sync count for this
        step too (three small launches per refresh, whatever the number of weights), so the weight roles' histories
        advance one real entry per refresh as on the per-module route, which folds its cached amax on every reuse."""
        snap = self._w_snap.get(arena)
        if snap is None:
            return
        idx = self._w_rows[arena]
        arena.parts.index_copy_(0, idx, torch.maximum(arena.parts.index_select(0, idx), snap))

    @classmethod
    def attach(cls, model: nn.Module, recipe: FP8Recipe, optimizer: "torch.optim.Optimizer | None" = None) -> "Fp8ParamSet":
        """The set of every ``FP8Linear`` under ``model``, quantised once now; with an optimizer, again after each
        of its steps."""
        ps = cls([m for m in model.modules() if isinstance(m, FP8Linear) and m.fp8_enabled], recipe)
        recipe._param_sets.add(ps)
        ps.sync()
        if optimizer is not None:
            ps.hook = optimizer.register_step_post_hook(lambda *_a, **_k: ps.sync())
        return ps
