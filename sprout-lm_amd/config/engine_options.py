"""Options of the serving engine (reference: EngineOptions, src/engine.ts:18-26, :55-65)."""
from __future__ import annotations

from dataclasses import dataclass, fields

from .base import ConfigError


@dataclass(frozen=True)
class EngineOptions:
    """Names and meanings follow the reference's EngineOptions, in snake_case.

    block_size          tokens in one cache page
    num_blocks          pages in every cache group's pool
    max_sequences       requests that may run at a time
    max_batch_tokens    token budget of one step
    prefill_chunk_size  most prompt tokens of one request in one step
    prefix_caching      share full prompt pages between requests
    record_trace        keep every event in `engine.trace`
    decode_lookahead    launch the next step of decoded tokens before the running one has been read back
                        (not in the reference; off: every step waits for its tokens first)
    step_token_multiple a step that would hold more tokens than this is cut back to a whole multiple of it, by
                        shortening the portion of a prompt that crosses the line (not in the reference; 1: off).
                        The tiled kernels work on blocks of up to 256 tokens: a step of 264 costs nearly as much
                        as one of 512.
    weight_limit_mib    most device memory the weights may take, in MiB (the reference's CUDA_WEIGHT_LIMIT_MIB;
                        0: no limit of their own)
    reserve_mib         device memory that must stay free once weights and cache pools are allocated, in MiB
                        (the reference's CUDA_RESERVE_MIB, default 1024 there as here); a model or pool that
                        does not fit is refused before anything is allocated
    strict_tensors      a checkpoint tensor that the model does not ask for is an error (off: left unread)
    """

    block_size: int = 16
    num_blocks: int = 256
    max_sequences: int = 64
    max_batch_tokens: int = 2048
    prefill_chunk_size: int = 512
    prefix_caching: bool = True
    record_trace: bool = False
    decode_lookahead: bool = True
    step_token_multiple: int = 1
    weight_limit_mib: int = 0
    reserve_mib: int = 1024
    strict_tensors: bool = False

    def __post_init__(self):
        for f in fields(self):
            value = getattr(self, f.name)
            if f.name in ("prefix_caching", "record_trace", "decode_lookahead", "strict_tensors"):
                if not isinstance(value, bool):
                    raise ConfigError(f"{f.name} must be a boolean.")
            elif f.name in ("weight_limit_mib", "reserve_mib"):
                if isinstance(value, bool) or not isinstance(value, int) or value < 0:
                    raise ConfigError(f"{f.name} must be a non-negative integer.")
            elif isinstance(value, bool) or not isinstance(value, int) or value <= 0:
                raise ConfigError(f"{f.name} must be a positive integer.")
