"""Learned RMSNorm (reference: norm, src/qwen.ts:72-77)."""
from __future__ import annotations

from .. import ops
from ..weights.loader import TensorSpec
from .base import Norm, NormFold, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    """y = x / sqrt(mean(x^2) + eps) * weight; sums in float32, the weight is used as it is."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, size: int, eps: float):
        self.size, self.eps = size, eps

    def tensors(self):
        return {"weight": TensorSpec((self.size,), "vector", "one_plus_normal")}

    def forward(self, ctx, x, out, rows=None):
        ops.rmsnorm(x, self.w["weight"], self.eps, out, rows)
        return out

    def fold(self):
        return NormFold("rms", self.w["weight"], self.eps)
