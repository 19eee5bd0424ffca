"""Dense gated feed-forward (reference: src/qwen.ts:196-200)."""
from __future__ import annotations

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import FeedForward, register_part


@register_part("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    """down(act(gate(x)) * up(x)), no biases.  gate and up are kept as one matrix [2 * inner, hidden]."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, inner: int, activation: str = "silu"):
        if activation not in ops.GATE_ACTIVATIONS:     # refused when the part is built, not at the first step
            raise ValueError(f"Gated feed-forward with activation {activation!r} has no kernel; "
                             f"there are kernels for {sorted(ops.GATE_ACTIVATIONS)}.")
        self.hidden, self.inner, self.activation = hidden, inner, activation

    def flops(self, tokens: int, pairs: int = 0) -> float:
        return 2.0 * tokens * 3 * self.hidden * self.inner

    def tensors(self):
        return {"gate_proj.weight": TensorSpec((self.inner, self.hidden)),
                "up_proj.weight": TensorSpec((self.inner, self.hidden)),
                "down_proj.weight": TensorSpec((self.hidden, self.inner))}

    def bind(self, tensors):
        self.w_gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.w_down = tensors["down_proj.weight"]
        self.w = {}

    def _fused(self, T: int, norm: bool) -> bool:
        return self.w_gate_up.dtype == torch.bfloat16 and ops.fused_supported(ops.FUSED_SILU, T, 2 * self.inner,
                                                                               self.hidden, norm=norm, variant=self.activation)

    fuse_input_norm = True    # see Attention.fuse_input_norm
    fuse_input_norm_f32 = True

    def forward_from_residual(self, ctx, norm, residual) -> bool:
        T = residual.shape[0]
        fold = norm.fold() if self.fuse_input_norm else None
        if fold is None or fold.kind != "rms":       # the one prologue the product kernels have
            return False
        if ctx.act_dtype == torch.float32 and self.fuse_input_norm_f32:
            act = ctx.buffer("gated", (T, self.inner), ctx.act_dtype)
            if not ops.gate_up_silu_f32(self.w_gate_up, residual, act, activation=self.activation, norm_weight=fold.weight,
                                        eps=fold.eps):
                return False
            ops.gemm(act, self.w_down, residual, accumulate=True)
            return True
        if ctx.act_dtype != torch.bfloat16 or T > 64 or not self._fused(T, True):
            return False
        if not ops.fused_norm_pays(T, 2 * self.inner, self.hidden):
            return False
        act = ctx.buffer("gated", (T, self.inner), ctx.act_dtype)
        ops.gate_up_silu(self.w_gate_up, act, residual=residual, norm_weight=fold.weight, eps=fold.eps,
                         activation=self.activation)
        ops.gemm(act, self.w_down, residual, accumulate=True)
        return True

    def forward(self, ctx, h, residual):
        T = h.shape[0]
        act = ctx.buffer("gated", (T, self.inner), ctx.act_dtype)
        if ctx.act_dtype == torch.bfloat16 and self._fused(T, False):
            ops.gate_up_silu(self.w_gate_up, act, x=h, activation=self.activation)
        elif ctx.act_dtype == torch.float32 and ops.gate_up_silu_f32(self.w_gate_up, h, act, activation=self.activation):
            pass
        else:
            gu = ctx.buffer("gate_up", (T, 2 * self.inner), ctx.act_dtype)
            ops.gemm(h, self.w_gate_up, gu)
            ops.silu_mul(gu, act, activation=self.activation)
        ops.gemm(act, self.w_down, residual, accumulate=True)
