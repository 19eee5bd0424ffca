"""Python faces of the HIP kernels.  Each takes torch tensors on the GPU, checks shapes on the host
and launches on torch's current stream."""
from .kernels import (FUSED_ROPE, FUSED_SILU, GATE_ACTIVATIONS, MAX_HEAD_DIM, ROTARY_PAIRINGS, SCORE_STAGES, AttentionBatch, check_attention_sizes, attention, attention_lists, attention_plan, mean_tile_walk,
                      feed_tokens, probe_machine, fused_norm_pays, fused_supported, pipe_plan, pipe_tiles, PLAN_STORE, PLAN_ACCUMULATE, PLAN_GATED, PLAN_ROTATING, gate_up_silu, gate_up_silu_f32, qkv_rope_cache, qkv_rope_cache_f32, embed, gemm, rmsnorm, rope_cache, rope_table, sample, random_fill,
                      sample_workspace_floats, silu_mul, stream_scope)
from .library import KernelError, library

__all__ = ["FUSED_ROPE", "FUSED_SILU", "GATE_ACTIVATIONS", "MAX_HEAD_DIM", "ROTARY_PAIRINGS", "SCORE_STAGES", "check_attention_sizes", "fused_norm_pays", "fused_supported", "pipe_plan", "pipe_tiles", "PLAN_STORE", "PLAN_ACCUMULATE", "PLAN_GATED", "PLAN_ROTATING", "gate_up_silu", "gate_up_silu_f32", "qkv_rope_cache", "qkv_rope_cache_f32", "AttentionBatch", "attention", "attention_lists", "attention_plan", "mean_tile_walk", "embed", "feed_tokens", "gemm", "rmsnorm", "rope_cache", "rope_table", "sample", "random_fill",
           "sample_workspace_floats", "silu_mul", "stream_scope", "KernelError", "library", "probe_machine"]
