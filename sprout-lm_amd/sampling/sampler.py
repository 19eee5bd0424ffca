"""Turns logits rows into token ids on the device."""
from __future__ import annotations

import torch

from .. import ops
from .params import SamplingParams


class NonFiniteLogits(RuntimeError):
    """A row of logits held NaN or infinity (reference: native/cuda-device.inc:250-257)."""


class Sampler:
    def __init__(self, device, vocab_size: int):
        self.device, self.vocab_size = device, vocab_size
        self._workspace = None
        self._out = None

    def _buffers(self, rows: int):
        need = ops.sample_workspace_floats(rows, self.vocab_size)
        if self._workspace is None or self._workspace.numel() < need:
            self._workspace = torch.empty(max(need, 1), dtype=torch.float32, device=self.device)
        if self._out is None or self._out.numel() < rows:
            self._out = torch.empty(max(rows, 64), dtype=torch.int32, device=self.device)
        return self._workspace, self._out[:rows]

    def sample_device(self, logits: torch.Tensor, params: list[SamplingParams], counters: list[int]) -> torch.Tensor:
        """int32 token ids on the device, one per row of `logits` (-1 marks a non-finite row)."""
        rows = logits.shape[0]
        workspace, out = self._buffers(rows)
        if any(p.temperature > 0 for p in params):
            temperature = torch.tensor([float(p.temperature) for p in params], dtype=torch.float32).to(self.device)
            seed = torch.tensor([p.seed for p in params], dtype=torch.int64).to(self.device)
            counter = torch.tensor(counters, dtype=torch.int32).to(self.device)
            ops.sample(logits, out, workspace, temperature, seed, counter)
        else:
            ops.sample(logits, out, workspace)
        return out

    def sample(self, logits: torch.Tensor, params: list[SamplingParams], counters: list[int]) -> list[int]:
        """Token ids on the host; only 4 bytes a row cross the bus."""
        if logits.shape[0] == 0:
            return []
        tokens = self.sample_device(logits, params, counters).tolist()
        if any(t < 0 or t >= self.vocab_size for t in tokens):
            raise NonFiniteLogits("Non-finite logits: the model produced NaN or infinity.")
        return tokens
