"""Rotary position encoding, half-split ("neox") pairing (reference: rope, src/qwen.ts:81-92)."""
from __future__ import annotations

import torch

from .base import PositionEncoding, register_part


@register_part("position", "rotary_neox")
class NeoxRotary(PositionEncoding):
    """Pair (d, d + rotary_dim/2) of a head turns by position * theta^(-2d / rotary_dim).

    The table of inverse frequencies is computed in float64 and kept in float32; angles, sines
    and cosines are float32 in the kernel.  For float32 models the part also keeps what the float32
    table lost (`inv_freq_tail`), and the kernel computes angle, sine and cosine in float64: a float32
    angle is off by up to position * 6e-8, more than every other rounding of that path together once
    positions reach the thousands.
    """

    graph_safe = True

    graph_safe_portions = True
    pairing = "halves"      # which dimensions turn together, as the kernels name it (ops.ROTARY_PAIRINGS)

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None):
        self.head_dim, self.theta = head_dim, theta
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {head_dim}.")
        self.inv_freq = None
        self.inv_freq_tail = None

    def prepare(self, device, dtype):
        d = torch.arange(0, self.rotary_dim, 2, dtype=torch.float64)
        exact = float(self.theta) ** (-d / self.rotary_dim)
        self.inv_freq = exact.to(torch.float32).to(device)
        if dtype == torch.float32:
            self.inv_freq_tail = (exact - exact.to(torch.float32).to(torch.float64)).to(torch.float32).to(device)

    def table(self, ctx) -> torch.Tensor:
        """(cosine, sine) of every token's angles, float32 [T, rotary_dim / 2, 2]: the same in every layer, so
        the first layer of a step that asks computes it and the others find it in the step's context."""
        from .. import ops
        key = ("rotary_neox", self.rotary_dim, float(self.theta))
        found = ctx.shared.get(key)
        if found is None:
            found = ctx.buffer(f"rotation_table_{self.rotary_dim}_{float(self.theta)!r}",
                               (ctx.n_tokens, self.rotary_dim // 2, 2), torch.float32)
            ops.rope_table(ctx.positions, self.inv_freq, found)
            ctx.shared[key] = found
        return found


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No position encoding: queries and keys are used as projected."""

    rotary_dim = 0
    pairing = "halves"      # nothing turns; the kernels are asked for the pairing they have

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, head_dim: int = 0):
        self.head_dim = head_dim
        self.inv_freq = None

    def prepare(self, device, dtype):
        self.inv_freq = torch.zeros(1, dtype=torch.float32, device=device)
