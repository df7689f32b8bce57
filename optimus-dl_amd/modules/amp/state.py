"""Process-wide FP8 state: which recipe is active, and the scaling-factor storage.

Counterpart of what the reference leaves to its third-party backend when it
enters ``te.pytorch.autocast(enabled=True, recipe=...)``
(optimus_dl/modules/amp/fp8.py:337-340,357-360): a global "FP8 is on, with this
recipe" flag that FP8 modules consult in forward, and the amax-history / scale
tensors that delayed scaling refreshes when the outermost context exits.

Design for one MI355X:
  * the active-recipe stack is a plain module global guarded by a lock, so the
    autograd worker thread sees the same state as the thread that entered the
    context (a thread-local would not); backward additionally carries its recipe
    in the autograd ``ctx`` and never depends on the ambient state;
  * all delayed-scaling roles of the modules that first ran under a recipe live in
    ONE arena per (recipe, device, direction): history [H, R], scale [R],
    scale_inv [R], parts [R, 512].  Casts fold their block maxima into the role's
    strip of partial maxima and hand back the inverse scale they used; a single small
    kernel per arena folds the strips into row 0 and refreshes every role of the
    model per step;
  * the scaling state belongs to the MODULES, as in the reference's backend (which
    keeps ``fp8_meta`` on each layer): a module finds its roles again by history
    length, formats and device, whatever recipe object is active.  The fresh recipe
    that an evaluation forward builds
    (optimus_dl/recipe/train/mixins/managers/evaluation_manager.py:98-144) therefore
    works with the scales that training arrived at and reserves nothing; a recipe
    that records into roles it did not reserve adopts their arena and refreshes it
    when its own context exits.
"""

from __future__ import annotations

import threading
from typing import TYPE_CHECKING

import torch

from ... import native

if TYPE_CHECKING:  # pragma: no cover
    from .fp8 import FP8Recipe

_lock = threading.RLock()
_stack: list["FP8Recipe"] = []


def push_recipe(recipe: "FP8Recipe") -> int:
    with _lock:
        _stack.append(recipe)
        return len(_stack)


def pop_recipe() -> int:
    with _lock:
        _stack.pop()
        return len(_stack)


def active_recipe() -> "FP8Recipe | None":
    with _lock:
        return _stack[-1] if _stack else None


def is_fp8_active() -> bool:
    return active_recipe() is not None


class ScalingMeta:
    """View of ``n`` consecutive roles of an arena; mirrors the attribute names
    (``amax_history``, ``scale``, ``scale_inv``) that the reference's own FP8 test
    inspects on its backend modules (tests/optim/test_fp8.py:609-625)."""

    def __init__(self, arena: "MetaArena", first: int, n: int):
        self.arena, self.first, self.n = arena, first, n
        self.first_record_epoch: int | None = None   # arena epoch at the first cast that recorded an amax here

    def note_record(self, store: "MetaStore") -> None:
        """A cast running under the recipe that owns ``store`` is about to record this step's amax in
        row 0 of the history: that recipe's context exit has to refresh this arena."""
        if self.first_record_epoch is None:
            self.first_record_epoch = self.arena.epoch
        self.arena.dirty = True
        if self.arena.owner is not store:
            store.adopted.add(self.arena)

    @property
    def trained(self) -> bool:
        """True once the scales have been refreshed from at least one recorded amax; until then
        these roles carry the initial scale 1."""
        return self.first_record_epoch is not None and self.arena.epoch > self.first_record_epoch

    @property
    def amax_history(self) -> torch.Tensor:          # [H, n] view; row 0 is filled by the refresh at the end of a step
        return self.arena.history[:, self.first:self.first + self.n]

    @property
    def pending_amax(self) -> torch.Tensor:          # [n]: amax per role of the step in progress (0 after a refresh)
        return self.arena.parts[self.first:self.first + self.n].amax(dim=1)

    @property
    def scale(self) -> torch.Tensor:
        return self.arena.scale[self.first:self.first + self.n]

    @property
    def scale_inv(self) -> torch.Tensor:
        return self.arena.scale_inv[self.first:self.first + self.n]

    def amax_slot(self, role: int) -> torch.Tensor:
        """Where the casts of the step in progress record the role's partial maxima (``native.AMAX_PARTS``
        floats); the refresh folds them into row 0 of the history and clears them."""
        return self.arena.parts[self.first + role]

    def scale_of(self, role: int) -> torch.Tensor:
        return self.arena.scale[self.first + role:self.first + role + 1]

    def scale_inv_of(self, role: int) -> torch.Tensor:
        return self.arena.scale_inv[self.first + role:self.first + role + 1]


class MetaArena:
    """history [H, cap], scale [cap], scale_inv [cap], fmt [cap], parts [cap, AMAX_PARTS] for one direction."""

    def __init__(self, device: torch.device, history_len: int, capacity: int, direction: str = "fwd", owner=None):
        self.device, self.H, self.capacity = device, history_len, capacity
        self.direction, self.owner = direction, owner
        self.history = torch.zeros((history_len, capacity), dtype=torch.float32, device=device)
        self.scale = torch.ones(capacity, dtype=torch.float32, device=device)
        self.scale_inv = torch.ones(capacity, dtype=torch.float32, device=device)
        self.fmt = torch.zeros(capacity, dtype=torch.int32, device=device)
        # partial maxima of the step in progress, AMAX_PARTS per role: the casts fold their block maxima into
        # many words instead of one (same-address atomics retire one at a time), the refresh reduces them
        self.parts = torch.zeros((capacity, native.AMAX_PARTS), dtype=torch.float32, device=device)
        self.used = 0
        self.dirty = False         # some cast wrote an amax since the last update
        self.epoch = 0             # bumped by every refresh of scale / scale_inv (they are updated in place)

    def reserve(self, fmts: list[int]) -> ScalingMeta | None:
        n = len(fmts)
        if self.used + n > self.capacity:
            return None
        first = self.used
        self.fmt[first:first + n] = torch.tensor(fmts, dtype=torch.int32, device=self.device)
        self.used += n
        return ScalingMeta(self, first, n)


class MetaStore:
    """All arenas of one recipe.  Arenas are never reallocated (modules hold views
    into them), a full one is followed by a new one.  ``adopted``: arenas reserved under
    another recipe into which a cast under this one has recorded an amax."""

    CAPACITY = 2048

    def __init__(self, history_len: int):
        self.history_len = history_len
        self.arenas: dict[tuple[str, str], list[MetaArena]] = {}
        self.adopted: set[MetaArena] = set()

    def reserve(self, device: torch.device, direction: str, fmts: list[int]) -> ScalingMeta:
        key = (str(device), direction)
        chain = self.arenas.setdefault(key, [])
        if chain:
            meta = chain[-1].reserve(fmts)
            if meta is not None:
                return meta
        chain.append(MetaArena(device, self.history_len, self.CAPACITY, direction, self))
        return chain[-1].reserve(fmts)

    def dirty_arenas(self, direction: str) -> list[MetaArena]:
        own = [a for (dev, d), chain in self.arenas.items() if d == direction for a in chain if a.dirty and a.used]
        return own + [a for a in self.adopted if a.direction == direction and a.dirty and a.used]


def tensor_version(t) -> int:
    """The tensor's in-place modification counter, or a fresh negative number for a tensor made under
    ``torch.inference_mode`` (those keep no counter): such a tensor then never matches a cached entry."""
    try:
        return t._version
    except RuntimeError:
        global _no_version
        _no_version -= 1
        return _no_version


_no_version = 0
