"""Grouped-query causal attention over the paged cache (reference: src/qwen.ts:167-195)."""
from __future__ import annotations

import math

import torch

from .. import ops
from ..cache.spec import PagedKVSpec
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import Mixer, register_part


@register_part("mixer", "attention")
class Attention(Mixer):
    """q, k, v projections, position encoding of q and k, cache write, attention, output projection.

    hidden, heads, kv_heads, head_dim: sizes.  qkv_bias / out_bias: whether the projections carry
    biases.  position: a PositionEncoding part.  window: None for all earlier keys, else how many
    of the latest keys a query sees.  own_kv False: the layer has no k/v projections and reads the
    cache slot that another layer writes.  page_tokens: tokens in a page of this layer's cache (None: the
    cache manager's own page size; else a divisor of it), e.g. small pages for a short window.

    The three input projections are kept as one matrix [(heads + 2 kv_heads) * head_dim, hidden]
    (rows of q, then k, then v), concatenated when the tensors are bound.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, heads: int, kv_heads: int, head_dim: int, position, qkv_bias: bool = True,
                 out_bias: bool = False, window: int | None = None, own_kv: bool = True, scale: float | None = None,
                 page_tokens: int | None = None, scores: str = "scaled_dot"):
        try:      # sizes no kernel takes are refused when the part is built, not at the first step
            ops.check_attention_sizes(heads, kv_heads, head_dim)
        except ops.KernelError as error:
            raise ConfigError(str(error)) from None
        if scores not in ops.SCORE_STAGES:      # a cap, a bias or sinks between q . k and the softmax: a kernel variant
            raise ConfigError(f"No attention kernel for score stage {scores!r}; there are kernels for: {sorted(ops.SCORE_STAGES)}.")
        self.scores = scores
        if head_dim % 2 and getattr(position, "rotary_dim", 0):
            raise ConfigError(f"A rotation needs an even head size, got {head_dim}.")
        self.hidden, self.heads, self.kv_heads, self.head_dim = hidden, heads, kv_heads, head_dim
        self.position, self.qkv_bias, self.out_bias = position, qkv_bias, out_bias
        self.window, self.own_kv, self.page_tokens = window, own_kv, page_tokens
        self.scale = 1.0 / math.sqrt(head_dim) if scale is None else scale

    def cache_spec(self):
        return PagedKVSpec(self.kv_heads, self.head_dim, self.window, self.page_tokens)

    def cache_elements_per_token(self) -> int:
        return 2 * self.kv_heads * self.head_dim

    def flops(self, tokens: int, pairs: int = 0) -> float:
        q, kv = self.heads * self.head_dim, (self.kv_heads * self.head_dim if self.own_kv else 0)
        projections = 2.0 * tokens * self.hidden * (q + 2 * kv) + 2.0 * tokens * q * self.hidden
        return projections + 4.0 * q * pairs          # scores and weighted values: two products over every pair

    def tensors(self):
        q, kv = self.heads * self.head_dim, self.kv_heads * self.head_dim
        names = [("q_proj", q)] + ([("k_proj", kv), ("v_proj", kv)] if self.own_kv else [])
        out = {}
        for name, rows in names:
            out[f"{name}.weight"] = TensorSpec((rows, self.hidden))
            if self.qkv_bias:
                out[f"{name}.bias"] = TensorSpec((rows,), "vector")
        out["o_proj.weight"] = TensorSpec((self.hidden, q))
        if self.out_bias:
            out["o_proj.bias"] = TensorSpec((self.hidden,), "vector")
        return out

    def bind(self, tensors):
        names = ["q_proj"] + (["k_proj", "v_proj"] if self.own_kv else [])
        self.w_qkv = torch.cat([tensors[f"{n}.weight"] for n in names], dim=0).contiguous()
        self.b_qkv = torch.cat([tensors[f"{n}.bias"] for n in names], dim=0).contiguous() if self.qkv_bias else None
        self.w_o = tensors["o_proj.weight"]
        self.b_o = tensors.get("o_proj.bias")
        self.w = {}

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def subparts(self):
        return [self.position]

    def _fused(self, T: int, cache, norm: bool) -> bool:
        """Whether a projection kernel with bias, rotation and cache write folded in takes this call."""
        return (self.own_kv and cache.writes and self.w_qkv.dtype == torch.bfloat16
                and ops.fused_supported(ops.FUSED_ROPE, T, self.w_qkv.shape[0], self.hidden, self.head_dim,
                                        self.position.rotary_dim, norm, variant=self.position.pairing))

    # Folding the norm into the projection kernel (up to 64 tokens) saves a launch; the kernel asks for the
    # residual rows before its weights, so the norm is computed while the weights are on their way.  Every
    # block of the kernel normalises its 16 tokens' rows by itself and every tile of 16 tokens reads the weights
    # again, so this pays for narrow models and few blocks only (the library says: `ops.fused_norm_pays`).
    fuse_input_norm = True

    def forward_from_residual(self, ctx, norm, residual, cache) -> bool:
        T = residual.shape[0]
        fold = norm.fold() if self.fuse_input_norm else None
        if fold is None or fold.kind != "rms":       # the one prologue the projection kernels have
            return False
        if ctx.act_dtype == torch.float32:
            return self._fused_f32(ctx, residual, residual, cache, fold)
        if ctx.act_dtype != torch.bfloat16 or T > 64 or not self._fused(T, cache, True):
            return False
        if not ops.fused_norm_pays(T, self.w_qkv.shape[0], self.hidden):
            return False
        q = ctx.buffer("q", (T, self.heads * self.head_dim), ctx.act_dtype)
        ops.qkv_rope_cache(self.w_qkv, self.b_qkv, q, ctx.positions, self.position.inv_freq, self.position.rotary_dim,
                           cache.slot_mapping, cache.k, cache.v, self.heads, self.kv_heads, self.head_dim,
                           residual=residual, norm_weight=fold.weight, eps=fold.eps, pairing=self.position.pairing)
        self._attend(ctx, q, self.heads * self.head_dim, residual, cache)
        return True

    def _fused_f32(self, ctx, x, residual, cache, fold=None) -> bool:
        """The float32 path's decode step: projections, bias, rotation and cache write in one kernel (and the norm,
        where `fold` is given and x is the residual).  False where that kernel does not take the call."""
        T = x.shape[0]
        if not (self.own_kv and cache.writes) or T > 16:
            return False
        q = ctx.buffer("q", (T, self.heads * self.head_dim), ctx.act_dtype)
        if not ops.qkv_rope_cache_f32(self.w_qkv, self.b_qkv, x, q, ctx.positions, self.position.inv_freq,
                                      getattr(self.position, "inv_freq_tail", None), self.position.rotary_dim,
                                      cache.slot_mapping, cache.k, cache.v, self.heads, self.kv_heads, self.head_dim,
                                      norm_weight=None if fold is None else fold.weight,
                                      eps=0.0 if fold is None else fold.eps, pairing=self.position.pairing):
            return False
        self._attend(ctx, q, self.heads * self.head_dim, residual, cache)
        return True

    def _attend(self, ctx, q, q_stride, residual, cache):
        T = q.shape[0]
        attn = ctx.buffer("attn", (T, self.heads * self.head_dim), ctx.act_dtype)
        # a step of decoded tokens only: the kernels may fold the projection into the merge of the key chunks
        project = (self.w_o, residual) if self.b_o is None else None
        if ops.attention(q, q_stride, cache.k, cache.v, cache.block_tables, ctx.attention, attn, self.heads,
                         self.kv_heads, self.head_dim, self.window, self.scale,
                         workspace=lambda n: ctx.buffer("attention_partials", (n,), torch.float32),
                         kind=ctx.attention_kind, project=project, scores=self.scores):
            return
        ops.gemm(attn, self.w_o, residual, bias=self.b_o, accumulate=True)

    def forward(self, ctx, h, residual, cache):
        T = h.shape[0]
        if ctx.act_dtype == torch.bfloat16 and self._fused(T, cache, False):
            q = ctx.buffer("q", (T, self.heads * self.head_dim), ctx.act_dtype)
            # many tokens: the sines and cosines are the same in every layer, computed once per step
            table = self.position.table(ctx) if T > 64 and hasattr(self.position, "table") else None
            ops.qkv_rope_cache(self.w_qkv, self.b_qkv, q, ctx.positions, self.position.inv_freq,
                               self.position.rotary_dim, cache.slot_mapping, cache.k, cache.v, self.heads,
                               self.kv_heads, self.head_dim, x=h, table=table, pairing=self.position.pairing)
            self._attend(ctx, q, self.heads * self.head_dim, residual, cache)
            return
        if ctx.act_dtype == torch.float32 and self._fused_f32(ctx, h, residual, cache):
            return
        nkv = self.kv_heads if (self.own_kv and cache.writes) else 0
        width = (self.heads + 2 * nkv) * self.head_dim
        qkv = ctx.buffer("qkv", (T, width), ctx.act_dtype)
        w, b = self.w_qkv, self.b_qkv
        if nkv == 0 and self.own_kv:   # a second call of the layer that only reads: q rows only
            w = w[: self.heads * self.head_dim]
            b = None if b is None else b[: self.heads * self.head_dim]
        ops.gemm(h, w, qkv, bias=b)
        ops.rope_cache(qkv, ctx.positions, self.position.inv_freq, self.position.rotary_dim, self.heads, nkv,
                       self.head_dim, cache.slot_mapping if nkv else None, cache.k if nkv else None,
                       cache.v if nkv else None,
                       inv_freq_tail=getattr(self.position, "inv_freq_tail", None) if qkv.dtype == torch.float32 else None,
                       pairing=self.position.pairing)
        self._attend(ctx, qkv, width, residual, cache)
