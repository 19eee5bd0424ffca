"""Arrangement of parts in a layer (reference: src/qwen.ts:164-202)."""
from __future__ import annotations

from .base import Block, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x += mixer(norm(x)); x += feed_forward(norm(x)).  The residual stream x is float32."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, mixer_norm, mixer, ffn_norm, ffn):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "ffn_norm": self.ffn_norm, "ffn": self.ffn}

    def forward(self, ctx, residual, caches):
        T, H = residual.shape
        cache = caches.get("mixer")
        h = ctx.buffer("normed", (T, H), ctx.act_dtype)
        if not self.mixer.forward_from_residual(ctx, self.mixer_norm, residual, cache):
            self.mixer_norm.forward(ctx, residual, h)
            self.mixer.forward(ctx, h, residual, cache)
        if not self.ffn.forward_from_residual(ctx, self.ffn_norm, residual):
            self.ffn_norm.forward(ctx, residual, h)
            self.ffn.forward(ctx, h, residual)
