"""Composition root: one call that loads a model folder and sizes an engine for it.

Reference: createRuntime (src/runtime.ts:27-66), which takes a model directory and a number of
context tokens and builds weights, cache and engine once before requests are accepted.
"""
from __future__ import annotations

from .config.engine_options import EngineOptions


class Runtime:
    """`engine` plus the reference's runtime fields: `name`, `stats()`, `close()`."""

    def __init__(self, engine, name: str):
        self.engine, self.name = engine, name

    def generate(self, prompt, max_new_tokens: int = 16, **sampling):
        """Stream of events of one request (queued, token ..., finished)."""
        return self.engine.stream(prompt, max_new_tokens, **sampling)

    def stats(self) -> dict:
        return self.engine.stats()

    def close(self) -> None:
        self.engine.close()


def create_runtime(model_directory: str, dtype: str = "bfloat16", max_context_tokens: int = 2048,
                   block_size: int = 16, max_sequences: int = 4, max_batch_tokens: int = 2048,
                   prefill_chunk_size: int = 512, prefix_caching: bool = True, record_trace: bool = False,
                   step_token_multiple: int = 1, weight_limit_mib: int = 0, reserve_mib: int = 1024,
                   strict_tensors: bool = False) -> Runtime:
    """`max_context_tokens` sizes the cache pool (the reference's KV_TOKENS): ceil(tokens / block_size) pages.
    A pool larger than one request can use is allowed: it serves several requests.  `weight_limit_mib` and
    `reserve_mib` are the reference's CUDA_WEIGHT_LIMIT_MIB and CUDA_RESERVE_MIB."""
    from .engine.engine import Engine
    if isinstance(max_context_tokens, bool) or not isinstance(max_context_tokens, int) or max_context_tokens < 1:
        raise ValueError("Invalid max_context_tokens.")
    options = EngineOptions(block_size=block_size, num_blocks=-(-max_context_tokens // block_size),
                            max_sequences=max_sequences, max_batch_tokens=max_batch_tokens,
                            prefill_chunk_size=prefill_chunk_size, prefix_caching=prefix_caching,
                            record_trace=record_trace, step_token_multiple=step_token_multiple,
                            weight_limit_mib=weight_limit_mib, reserve_mib=reserve_mib, strict_tensors=strict_tensors)
    engine = Engine.from_folder(model_directory, dtype, options)
    return Runtime(engine, f"{model_directory} ({engine.model.plan.architecture}, {dtype}, HIP forward + device KV)")
