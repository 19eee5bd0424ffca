"""Token embedding and output head (reference: src/qwen.ts:162-163, :203)."""
from __future__ import annotations

from .. import ops
from ..weights.loader import TensorSpec
from .base import Part, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    graph_safe = True
    graph_safe_portions = True

    def __init__(self, vocab: int, hidden: int):
        self.vocab, self.hidden = vocab, hidden

    def tensors(self):
        return {"weight": TensorSpec((self.vocab, self.hidden))}

    def forward(self, ctx, tokens, residual):
        ops.embed(self.w["weight"], tokens, residual)

    def weight_elements(self) -> int:
        return 0      # a step gathers one row per token: nothing beside the matrices


@register_part("head", "linear_head")
class LinearHead(Part):
    """logits = W . x in float32.  With `tied`, W is the embedding table and the head has no tensor."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, vocab: int, hidden: int, tied: bool):
        self.vocab, self.hidden, self.tied = vocab, hidden, tied
        self.table = None

    def tensors(self):
        return {} if self.tied else {"weight": TensorSpec((self.vocab, self.hidden))}

    def bind(self, tensors):
        self.w = tensors
        if not self.tied:
            self.table = tensors["weight"]

    def tie(self, embedding_table):
        self.table = embedding_table

    def forward(self, ctx, h, logits):
        ops.gemm(h, self.table, logits)

    def weight_elements(self) -> int:
        return self.vocab * self.hidden      # the output matrix is read whole, also where it is the embedding table

    def flops(self, tokens: int, pairs: int = 0) -> float:
        return 2.0 * tokens * self.vocab * self.hidden
