"""Per-request sampling options."""
from __future__ import annotations

import math
from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    """temperature 0 is greedy (the reference's only mode, src/runner.ts:38-42); with a temperature
    above 0 the draw depends on (seed, output index) alone, not on what else runs beside the request.
    stop_token_ids None: the model's end-of-sequence ids.  ignore_eos: run to max_new_tokens."""

    temperature: float = 0.0
    seed: int = 0
    stop_token_ids: tuple[int, ...] | None = None
    ignore_eos: bool = False

    def __post_init__(self):
        if isinstance(self.temperature, bool) or not isinstance(self.temperature, (int, float)) \
                or not math.isfinite(self.temperature) or self.temperature < 0:
            raise ValueError("temperature must be a finite number >= 0.")
        if isinstance(self.seed, bool) or not isinstance(self.seed, int) or not 0 <= self.seed < 2 ** 63:
            raise ValueError("seed must be an integer in [0, 2^63).")
