"""Interfaces of the parts a model is put together from, and the registries that name them.

A part knows its own sizes and constants (constructor parameters), the tensors it needs (local
names, `tensors()`), and how to run on a step's batch (`forward`).  It does not know which model
it is in, which layer it is, or what its tensors are called in a checkpoint: the model plan gives
every part a name prefix, and the runner hands it its tensors under their local names.
"""
from __future__ import annotations

from typing import Callable

from ..weights.loader import TensorSpec

_REGISTRIES: dict[str, dict[str, type]] = {
    "mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {}, "embedding": {}, "head": {},
}


def register_part(category: str, name: str) -> Callable[[type], type]:
    """Class decorator: make `cls` available to model plans as part `name` of `category`."""
    if category not in _REGISTRIES:
        raise KeyError(f"Unknown part category {category!r}; categories are {sorted(_REGISTRIES)}.")

    def wrap(cls: type) -> type:
        _REGISTRIES[category][name] = cls
        cls.kind = name
        return cls

    return wrap


def make_part(category: str, name: str, **params):
    try:
        cls = _REGISTRIES[category][name]
    except KeyError:
        raise KeyError(f"No {category} part named {name!r}; registered: {sorted(_REGISTRIES[category])}.") from None
    return cls(**params)


def registered_parts(category: str) -> list[str]:
    return sorted(_REGISTRIES[category])


class Part:
    """Base of every part."""

    kind = ""
    # True if `forward` only launches work on the current stream from device-resident inputs (no
    # host-side decisions from the step's values, no allocation): such a part may be recorded into
    # a HIP graph and replayed with new values in the same buffers.
    graph_safe = False
    # True if that holds for every step, also one with portions of prompts in it (then `ctx.host` is empty).
    graph_safe_portions = False

    def tensors(self) -> dict[str, TensorSpec]:
        """Local tensor name -> what is expected of it."""
        return {}

    def bind(self, tensors: dict) -> None:
        """Receive the device tensors named in `tensors()`.  Called once after loading."""
        self.w = tensors

    def prepare(self, device, dtype) -> None:
        """Build device-side constants (tables of frequencies and the like).  Called once."""

    def subparts(self) -> list:
        """Parts that this part holds and runs itself (a mixer's position encoding): they are asked for
        `graph_safe` along with it."""
        return []

    def cache_spec(self):
        """What the part keeps between steps: a PagedKVSpec, a StateSpec, a dict of several of them by a name of
        the part's choosing (pages and a state of fixed size, say), or None.  Any part of a block may keep
        something; it receives the view of its slot (or a dict of views under the same names) from the block."""
        return None

    def cache_elements_per_token(self) -> int:
        """Cache elements that a decoded token reads per token of its context (keys and values)."""
        return 0

    # What a part costs, for measurement: the engine's bench adds these up over the model's parts and
    # knows no architecture.
    def weight_elements(self) -> int:
        """Elements of the part's tensors that one step reads (every weight once, whatever the batch)."""
        total = 0
        for spec in self.tensors().values():
            count = 1
            for n in spec.shape:
                count *= n
            total += count
        return total

    def flops(self, tokens: int, pairs: int = 0) -> float:
        """Floating-point operations of `forward` on `tokens` tokens (a multiply-add counts two).  `pairs`: the
        number of (query, key) pairs of the step, for parts that mix tokens.  Matrix products only."""
        return 0.0


class Norm(Part):
    def forward(self, ctx, x, out, rows=None):
        """out = norm(x[rows] or x).  x is the float32 residual stream, out has the activation dtype."""
        raise NotImplementedError

    def fold(self):
        """How the norm can be computed inside the kernel of the product that follows it, or None if it
        cannot: a `NormFold` whose `kind` names a prologue that the product kernels have.  A part that
        folds asks the norm, not its class."""
        return None


class NormFold:
    """A norm as a product kernel's prologue.  kind "rms": x * rsqrt(mean(x^2) + eps) * weight."""

    def __init__(self, kind: str, weight, eps: float):
        self.kind, self.weight, self.eps = kind, weight, eps


class PositionEncoding(Part):
    """Turns positions into something a mixer applies to its queries and keys.

    A rotary part provides `inv_freq` (float32 [rotary_dim / 2] on the device after `prepare`), `rotary_dim`
    (0: nothing turns) and `pairing`: which dimensions turn together, by the name the kernels know it under
    (`ops.ROTARY_PAIRINGS`; a pairing without a kernel is refused when the step is launched)."""

    rotary_dim = 0
    pairing = "halves"


class Mixer(Part):
    """Mixes information between the tokens of a sequence (attention, or anything with state)."""

    def forward(self, ctx, h, residual, cache):
        """residual += mixer(h).  `cache` is this call's cache slot view (engine.batch.CacheSlotView), a dict of
        views if `cache_spec` names several, or None."""
        raise NotImplementedError

    def forward_from_residual(self, ctx, norm, residual, cache) -> bool:
        """Optional shortcut: residual += mixer(norm(residual)) with the norm folded into the mixer's
        first kernel.  Returns False (and does nothing) where the mixer has no such kernel."""
        return False


class FeedForward(Part):
    def forward(self, ctx, h, residual):
        """residual += feed_forward(h), token by token."""
        raise NotImplementedError

    def forward_from_residual(self, ctx, norm, residual) -> bool:
        """Optional shortcut, as Mixer.forward_from_residual."""
        return False


class Block(Part):
    """Arranges mixers, feed-forwards and their norms around the residual stream."""

    def parts(self) -> dict[str, Part]:
        """The block's parts by the names under which the model plan gave them; everything the engine wants of a
        block's parts (tensors, cache needs, costs, whether they may be recorded) it asks through this."""
        raise NotImplementedError

    def forward(self, ctx, residual, caches: dict):
        """Run the block on the step's tokens.  `caches`: part name -> what that part's `cache_spec` asked for in
        this call of the run order (a view, or a dict of views); parts that keep nothing are absent."""
        raise NotImplementedError
