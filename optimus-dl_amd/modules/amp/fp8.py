"""FP8 recipe and autocast contexts, backed by the MI355X kernels.

API-compatible with optimus_dl/modules/amp/fp8.py: the enums (:40-61), the
string parsers (:96-147) with their error texts, ``Fp8RecipeConfig`` (:151),
``FP8Recipe`` with its constructor arguments echoed as attributes, ``.recipe``,
``.autocast()`` and ``.backward()`` (:180-360), ``create_fp8_recipe`` (:387),
``fp8_autocast`` (:450) and ``fp8_backward`` (:501).

Where the reference hands the recipe to a third-party CUDA library, this module
owns the scaling policy itself:

  tensorwise  amax of the tensor at hand -> scale -> cast       (two passes)
  delayed     cast with the scale from the amax history while recording this
              step's amax; histories roll and scales refresh when the outermost
              autocast / backward context exits                 (one pass)
  rowwise     (extension, no reference enum) one scale per row of each operand
              along its non-contracted axis
  mxfp8       OCP microscaling: 32-element blocks along the contraction axis,
              one E8M0 scale byte each, applied by the MFMA      (one pass)
  blockwise   1 x 128 blocks (activations, gradients) and 128 x 128 blocks
              (weights) with power-of-two scales, same GEMM      (one pass)
"""

from __future__ import annotations

import logging
import weakref
from collections.abc import Iterator
from contextlib import contextmanager
from dataclasses import dataclass
from enum import Enum
from typing import Any

import torch

from ... import native
from . import state as _state

logger = logging.getLogger(__name__)
_logged_once: set[str] = set()


def _info_once(msg: str) -> None:
    if msg not in _logged_once:
        _logged_once.add(msg)
        logger.info(msg)


class Fp8Format(Enum):
    HYBRID = "hybrid"   # E4M3 forward, E5M2 gradients
    E4M3 = "e4m3"
    E5M2 = "e5m2"


class Fp8RecipeType(str, Enum):
    DELAYED = "delayed"
    TENSORWISE = "tensorwise"
    BLOCKWISE = "blockwise"
    MXFP8 = "mxfp8"
    ROWWISE = "rowwise"   # extension: per-row / per-output-channel scales


_FORMAT_ALIASES = {
    Fp8Format.HYBRID: ("hybrid", "hybrid_fp8", "fp8_hybrid"),
    Fp8Format.E4M3: ("e4m3", "fp8_e4m3", "e4m3fn", "float8_e4m3fn"),
    Fp8Format.E5M2: ("e5m2", "fp8_e5m2", "e5m2fn", "float8_e5m2"),
}
_RECIPE_ALIASES = {
    Fp8RecipeType.DELAYED: ("delayed", "delayed_scaling"),
    Fp8RecipeType.TENSORWISE: ("tensorwise", "tensor_wise", "current", "current_scaling"),
    Fp8RecipeType.BLOCKWISE: ("blockwise", "block_wise", "float8_block"),
    Fp8RecipeType.MXFP8: ("mxfp8", "mxfp8_block"),
    Fp8RecipeType.ROWWISE: ("rowwise", "row_wise", "channelwise"),
}


def is_native_backend_available() -> bool:
    """True when the compiled kernel library is present and a GPU is visible."""
    return native.is_built() and torch.cuda.is_available()


def is_transformer_engine_available() -> bool:
    """Name kept for drop-in use: "is an FP8 backend available?"  Here the backend
    is the in-tree HIP library rather than the CUDA package the reference probes
    for (fp8.py:64-77)."""
    return is_native_backend_available()


def get_transformer_engine_version() -> str | None:
    if not is_native_backend_available():
        return None
    from ... import __version__

    return f"odl-fp8-{__version__}"


def get_fp8_format_from_string(format_str: str) -> Fp8Format:
    key = format_str.lower()
    for fmt, names in _FORMAT_ALIASES.items():
        if key in names:
            return fmt
    raise ValueError(f"Unknown FP8 format: {key}. Supported formats: hybrid, e4m3, e5m2")


def get_fp8_recipe_type_from_string(recipe_str: str) -> Fp8RecipeType:
    key = recipe_str.lower()
    for rt, names in _RECIPE_ALIASES.items():
        if key in names:
            return rt
    raise ValueError(f"Unknown FP8 recipe type: {key}. Supported types: delayed, tensorwise, blockwise, mxfp8")


@dataclass
class Fp8RecipeConfig:
    recipe_type: str = "delayed"
    format: str = "hybrid"
    margin: int = 0
    amax_history_len: int = 1024
    amax_compute_algo: str = "max"
    reduce_amax: bool = True
    fp8_dpa: bool = False
    fp8_mha: bool = False


@dataclass(frozen=True)
class ScalingPolicy:
    """What ``FP8Recipe.recipe`` returns: the resolved policy the kernels follow."""

    kind: str                 # "delayed" | "tensorwise" | "rowwise" | "mxfp8" | "blockwise"
    fmt_fwd: int              # native.E4M3 / native.E5M2 for activations and weights
    fmt_bwd: int              # ... for gradients
    margin: int
    amax_history_len: int
    amax_compute_algo: str    # "max" | "most_recent"
    reduce_amax: bool         # one GPU: the cross-rank MAX all-reduce is a no-op
    mx_scale_rule: int = 1    # mxfp8 only: native.MX_CEIL (shared exponent rounded up) or native.MX_FLOOR (OCP formula)


class FP8Recipe:
    """Scaling recipe + the contexts that switch FP8 on for the Linear modules."""

    def __init__(
        self,
        recipe_type: str | Fp8RecipeType = Fp8RecipeType.DELAYED,
        format: str | Fp8Format = Fp8Format.HYBRID,
        margin: int = 0,
        amax_history_len: int = 1024,
        amax_compute_algo: str = "max",
        reduce_amax: bool = True,
        fp8_dpa: bool = False,
        fp8_mha: bool = False,
        wgrad: bool = True,
        mx_scale_rule: str = "ceil",
    ):
        if not is_native_backend_available():
            raise ImportError(
                "The FP8 kernel library (libodl_fp8.so) and a visible MI355X are required for FP8 training. "
                "Build the library with: python -m optimus_dl_amd.build"
            )
        if torch.cuda.is_available():
            native.init_device()      # per-device look-ups of the library, which must not happen under graph capture
        self.recipe_type = get_fp8_recipe_type_from_string(recipe_type) if isinstance(recipe_type, str) else recipe_type
        self.format = get_fp8_format_from_string(format) if isinstance(format, str) else format
        self.margin = margin
        self.amax_history_len = amax_history_len
        self.amax_compute_algo = amax_compute_algo
        self.reduce_amax = reduce_amax
        self.fp8_dpa = fp8_dpa
        self.fp8_mha = fp8_mha
        self.wgrad = wgrad

        if self.format == Fp8Format.HYBRID:
            fwd, bwd = native.E4M3, native.E5M2
        elif self.format == Fp8Format.E4M3:
            fwd, bwd = native.E4M3, native.E4M3
        elif self.format == Fp8Format.E5M2:
            if self.recipe_type == Fp8RecipeType.DELAYED:
                raise ValueError(
                    "Pure E5M2 format is not supported by delayed recipe. Please use 'hybrid' or 'e4m3' format instead."
                )
            fwd, bwd = native.E5M2, native.E5M2
        else:
            raise ValueError(f"Unsupported FP8 format: {self.format}")
        if amax_compute_algo not in ("max", "most_recent"):
            raise ValueError(f"Unsupported amax_compute_algo: {amax_compute_algo} (max, most_recent)")
        if amax_history_len < 1:
            raise ValueError("amax_history_len must be >= 1")
        # mxfp8: how a block's shared exponent follows from its amax.  "ceil" (default): ceil(log2(amax / fp8_max)),
        # nothing saturates -- what a quantiser gives that converts amax / fp8_max to E8M0 rounding up, as the backend
        # behind the reference's `recipe: mxfp8` (fp8.py:301-306) is published to.  "floor": the formula of the OCP MX
        # specification, floor(log2 amax) - emax, which lets a block amax in the top eighth of its binade saturate.
        if mx_scale_rule not in ("ceil", "floor"):
            raise ValueError(f"Unsupported mx_scale_rule: {mx_scale_rule} (ceil, floor)")
        self.mx_scale_rule = mx_scale_rule
        self._recipe = ScalingPolicy(
            kind=self.recipe_type.value, fmt_fwd=fwd, fmt_bwd=bwd, margin=margin,
            amax_history_len=amax_history_len, amax_compute_algo=amax_compute_algo, reduce_amax=reduce_amax,
            mx_scale_rule=native.MX_CEIL if mx_scale_rule == "ceil" else native.MX_FLOOR,
        )
        # the arenas that modules reserve their delayed-scaling roles in when they first run under this recipe.
        # The modules keep the views (the state is theirs): another recipe of the same shape -- the one an
        # evaluation forward builds -- finds the roles on the module and reserves nothing here
        self._store = _state.MetaStore(amax_history_len)
        self._depth = 0
        # the last activation quantised under this recipe, so that Linears fed by the same tensor
        # (gate/up, q/k/v) quantise it once; dropped when the outermost context is left
        self.shared_input: dict[str, Any] | None = None
        self.share_inputs = True
        # quantised weights are kept while the Parameter's version counter stands still (microbatches of one
        # optimizer step).  Code that rewrites weights through ``param.data`` does not move that counter:
        # set this to False there, and every forward quantises its weight again (what the reference does).
        self.cache_weights = True
        # wgrad reads the row-major codes of dy with the tokens as the slow axis where the shapes allow
        # (no transposed copy of dy); False keeps the cast+transpose route everywhere
        self.direct_layouts = True
        # partial maxima handed over by the kernel that produced a tensor (SwiGLU, RMSNorm), so that
        # the Linear that quantises this very tensor skips its amax pass; a handful of entries
        self.producer_parts: list[tuple[tuple, torch.Tensor, torch.Tensor]] = []
        # Linears fed by one tensor (q/k/v, gate/up) run as one autograd node whose data gradients are summed by the
        # GEMMs' accumulate flag (modules/fp8_linear.py: linear_group, SiblingGroup); False: every Linear on its own
        self.fuse_dgrad_sum = True
        # ... and by ONE GEMM that runs its contraction through all members' operands where the shapes allow
        # (native.gemm_nt_sum: no read-modify-write of dx per further member); False: always the accumulate flag
        self.fuse_dgrad_gemm = True
        self._sibling_groups: "weakref.WeakSet" = weakref.WeakSet()
        # Gradient accumulation over microbatches (the reference's acc_steps > 1): with this set, a weight gradient is
        # added straight into an existing ``weight.grad`` by the GEMM and autograd is handed None for it, instead
        # of a separate ``grad += dw`` pass per weight and microbatch.  Off by default: tensor hooks on the weight's
        # gradient (DDP / FSDP reducers) do not see a gradient that never passes through autograd.
        self.fuse_wgrad_accumulation = False
        # Members of such a group whose weight gradients are each a GEMM of few tiles over a transposed copy of dy (k and v
        # of a grouped-query attention block) get them from ONE GEMM over their transposed codes side by side; the
        # gradients are then row ranges of one matrix.  False: a GEMM per member
        self.fuse_sibling_wgrad = True
        # Fp8ParamSets attached under this recipe (delayed scaling: they re-record their weights' maxima at each refresh)
        self._param_sets: "weakref.WeakSet" = weakref.WeakSet()
        _info_once(
            f"Created FP8 recipe with format={self.format.value}, amax_history_len={amax_history_len}, "
            f"amax_compute_algo={amax_compute_algo}"
        )

    # ------------------------------------------------------------------ policy
    @property
    def recipe(self) -> ScalingPolicy:
        return self._recipe

    @property
    def is_delayed(self) -> bool:
        return self._recipe.kind == "delayed"

    def reserve_meta(self, device: torch.device, direction: str, fmts: list[int]) -> "_state.ScalingMeta":
        return self._store.reserve(device, direction, fmts)

    def update_scales(self, direction: str) -> None:
        """Roll the histories of every role that saw a cast since the last update
        and refresh their scales: one small kernel per arena."""
        if not self.is_delayed:
            return
        algo = native.AMAX_MAX if self.amax_compute_algo == "max" else native.AMAX_MOST_RECENT
        for arena in self._store.dirty_arenas(direction):
            if direction == "fwd":
                for ps in self._param_sets:
                    ps.refold(arena)
            R = arena.used
            native.delayed_update_raw(arena.history, arena.H, arena.capacity, R, arena.scale, arena.scale_inv,
                                      arena.fmt, self.margin, algo, amax_parts=arena.parts)
            arena.dirty = False
            arena.epoch += 1

    # ------------------------------------------------------- fp8.param
    def attach_params(self, model: torch.nn.Module, optimizer: "torch.optim.Optimizer | None" = None):
        """``fp8.param: true`` (optimus_dl/modules/optim/config.py:36-37): keep the weights of the model's FP8
        Linears quantised between optimizer steps.  All of them are quantised in one or two launches now and, when
        the optimizer is given, after each of its steps (a step post-hook); the forwards in between launch nothing
        for the weights.  Returns the ``Fp8ParamSet`` (call its ``sync()`` yourself after a step when no optimizer
        was given), or None for the rowwise recipe, which keeps the per-module route."""
        from ..fp8_linear import Fp8ParamSet

        if self._recipe.kind not in ("tensorwise", "delayed"):
            _info_once(f"fp8.param: the '{self._recipe.kind}' recipe quantises each weight in its own module (cached per parameter "
                       "version); nothing to attach")
            return None
        return Fp8ParamSet.attach(model, self, optimizer)

    # ---------------------------------------------------------- checkpointing
    _DIRECTIONS = (("fwd", "scaling_fwd"), ("bwd", "scaling_bwd"))

    @staticmethod
    def _fp8_modules(model: torch.nn.Module):
        return [(name, mod) for name, mod in model.named_modules() if hasattr(mod, "_meta") and hasattr(mod, "fp8_meta")]

    def state_dict(self, model: torch.nn.Module) -> dict:
        """Delayed-scaling state (amax histories, scales) of every FP8 module of ``model``, as CPU
        tensors keyed by the module's qualified name.  The state lives with the modules, but it is not
        part of ``model.state_dict()`` (whose keys stay those of the plain model): a trainer that
        checkpoints a delayed-scaling run saves this dict next to the model's and hands it to
        :meth:`load_state_dict` after building model and recipe, before the first step.  Empty for
        the recipes that keep no state between steps (tensorwise, rowwise)."""
        out: dict[str, Any] = {"format_version": 1, "amax_history_len": self.amax_history_len, "modules": {}}
        if not self.is_delayed:
            return out
        for name, mod in self._fp8_modules(model):
            entry = {}
            for direction, _ in self._DIRECTIONS:
                meta = mod._meta(self, mod.weight.device, direction)
                entry[direction] = {"amax_history": meta.amax_history.detach().cpu().clone(),
                                    "scale": meta.scale.detach().cpu().clone(),
                                    "scale_inv": meta.scale_inv.detach().cpu().clone(),
                                    "trained": meta.trained}
            out["modules"][name] = entry
        return out

    def load_state_dict(self, model: torch.nn.Module, state: dict, strict: bool = True) -> None:
        """Restore what :meth:`state_dict` saved.  The roles of every module are reserved here, so the
        call works on a freshly built model that has not run a forward yet.  Quantised weights cached
        under other scales are invalidated (an attached ``Fp8ParamSet`` casts its weights again, so the order
        "load the weights, attach the set, load this state" resumes on the codes of the uninterrupted run).  strict: module names that are in ``state`` and not in the
        model, or the reverse, raise ``KeyError``."""
        if not self.is_delayed:
            return
        if state.get("amax_history_len", self.amax_history_len) != self.amax_history_len:
            raise ValueError(f"amax_history_len of the checkpoint ({state.get('amax_history_len')}) differs from this "
                             f"recipe's ({self.amax_history_len})")
        saved = state.get("modules", {})
        mods = dict(self._fp8_modules(model))
        if strict:
            missing, unexpected = sorted(set(mods) - set(saved)), sorted(set(saved) - set(mods))
            if missing or unexpected:
                raise KeyError(f"FP8 scaling state does not match the model: no state for {missing}, no module for {unexpected}")
        touched: set = set()
        for name, entry in saved.items():
            mod = mods.get(name)
            if mod is None:
                continue
            for direction, _ in self._DIRECTIONS:
                blob = entry[direction]
                meta = mod._meta(self, mod.weight.device, direction)
                touched.add(meta.arena)
                if tuple(blob["amax_history"].shape) != tuple(meta.amax_history.shape):
                    raise ValueError(f"{name}/{direction}: saved history {tuple(blob['amax_history'].shape)} does not fit "
                                     f"{tuple(meta.amax_history.shape)}")
                meta.amax_history.copy_(blob["amax_history"])
                meta.scale.copy_(blob["scale"])
                meta.scale_inv.copy_(blob["scale_inv"])
                if blob.get("trained", True):
                    meta.first_record_epoch = -1
        for arena in touched:          # codes made under the old scales are stale
            arena.epoch += 1
        # ... including the codes an Fp8ParamSet keeps per optimizer step (made at whatever scale was in force at
        # its last sync, e.g. the initial scale 1 of a freshly attached set): they are dropped, and the sets attached
        # under this recipe cast their weights again now, under the restored scales
        for mod in mods.values():
            cache = getattr(mod, "_wcache", None)
            if cache is not None:
                cache.kept = None
                cache.key = None
        for ps in list(self._param_sets):
            ps.sync()

    # ------------------------------------------------------- producer hand-over
    @staticmethod
    def _tensor_key(t: torch.Tensor) -> tuple:
        return (t.data_ptr(), _state.tensor_version(t), t.numel(), t.dtype, t.device)

    def offer_parts(self, tensor: torch.Tensor, parts: torch.Tensor) -> None:
        """Record the partial maxima of |tensor| that its producer computed.  The entry keeps the
        tensor alive (its address cannot be reused meanwhile); an in-place change bumps the
        version and the entry no longer matches."""
        if self._recipe.kind != "tensorwise":
            return
        self.producer_parts.append((self._tensor_key(tensor), tensor, parts))
        if len(self.producer_parts) > 8:
            del self.producer_parts[0]

    def take_parts(self, tensor: torch.Tensor) -> torch.Tensor | None:
        """Partial maxima for exactly this tensor (or a view of all of it), if a producer left them."""
        if not self.producer_parts:
            return None
        key = self._tensor_key(tensor)
        for i, (k, _, parts) in enumerate(self.producer_parts):
            if k == key:
                del self.producer_parts[i]
                return parts
        return None

    # ---------------------------------------------------------------- contexts
    @contextmanager
    def autocast(self) -> Iterator[None]:
        """Forward context: FP8 Linears quantise while it is active.  Leaving the
        outermost one refreshes the forward scales (delayed scaling)."""
        _state.push_recipe(self)
        self._depth += 1
        try:
            yield
        finally:
            self._depth -= 1
            _state.pop_recipe()
            if self._depth == 0:
                self.shared_input = None
                self.producer_parts.clear()
                for grp in list(self._sibling_groups):      # outputs made for siblings that were never asked for
                    grp.clear()
                self._sibling_groups.clear()
                self.update_scales("fwd")
                # gradients recorded by a backward that ran outside any backward()
                # context are folded in here, one step late but never lost
                self.update_scales("bwd")

    @contextmanager
    def backward(self) -> Iterator[None]:
        """Backward context: leaving it refreshes the gradient scales."""
        _state.push_recipe(self)
        self._depth += 1
        try:
            yield
        finally:
            self._depth -= 1
            _state.pop_recipe()
            if self._depth == 0:
                self.shared_input = None          # a forward recomputed by activation checkpointing may have left one
                self.producer_parts.clear()
                for grp in list(self._sibling_groups):
                    grp.clear()
                self._sibling_groups.clear()
                self.update_scales("bwd")

    def prepare_for_backward(self, *args: Any, **kwargs: Any) -> tuple[Any, ...]:
        return args

    def prepare(self, *args: Any, **kwargs: Any) -> tuple[Any, ...]:
        return args


def create_fp8_recipe(
    recipe_type: str | Fp8RecipeType = Fp8RecipeType.DELAYED,
    format: str | Fp8Format = Fp8Format.HYBRID,
    margin: int = 0,
    amax_history_len: int = 1024,
    amax_compute_algo: str = "max",
    reduce_amax: bool = True,
    fp8_dpa: bool = False,
    fp8_mha: bool = False,
    wgrad: bool = True,
    mx_scale_rule: str = "ceil",
) -> FP8Recipe | None:
    """FP8Recipe when the backend is usable, else None (callers fall back to bf16 AMP)."""
    if not is_native_backend_available():
        logger.warning(
            "FP8 backend not available (libodl_fp8.so missing or no GPU). FP8 training will be disabled. "
            "Build with: python -m optimus_dl_amd.build"
        )
        return None
    return FP8Recipe(recipe_type=recipe_type, format=format, margin=margin, amax_history_len=amax_history_len,
                     amax_compute_algo=amax_compute_algo, reduce_amax=reduce_amax, fp8_dpa=fp8_dpa, fp8_mha=fp8_mha,
                     wgrad=wgrad, mx_scale_rule=mx_scale_rule)


@contextmanager
def fp8_autocast(device: torch.device, fp8_recipe: FP8Recipe | None, enabled: bool = True,
                 dtype: torch.dtype | None = None) -> Iterator[None]:
    """FP8 autocast outside, ordinary AMP autocast inside (for everything that is
    not an FP8 Linear); plain AMP when there is no recipe or no GPU."""
    if not enabled:
        yield
        return
    if dtype is None:
        dtype = torch.bfloat16
    if fp8_recipe is not None and device.type == "cuda":
        with fp8_recipe.autocast():
            with torch.autocast(device.type, dtype=dtype, enabled=True):
                yield
    else:
        with torch.autocast(device.type, dtype=dtype, enabled=True):
            yield


@contextmanager
def fp8_backward(fp8_recipe: FP8Recipe | None, enabled: bool = True) -> Iterator[None]:
    if not enabled or fp8_recipe is None:
        yield
        return
    with fp8_recipe.backward():
        yield
