"""Shared pieces of the tests: the tiny configurations, model folders, and the two sides compared."""
from __future__ import annotations

import functools
import json
import os

import numpy as np
import torch

from tests.plain import qwen2_plain as P

# Two tiny Qwen2 configurations that differ in every size and option.
TINY_A = dict(model_type="qwen2", hidden_act="silu", hidden_size=64, intermediate_size=128, num_hidden_layers=2,
              num_attention_heads=4, num_key_value_heads=2, vocab_size=256, max_position_embeddings=128,
              rms_norm_eps=1e-6, rope_theta=10000.0, tie_word_embeddings=True, eos_token_id=255)
TINY_B = dict(model_type="qwen2", hidden_act="silu", hidden_size=96, intermediate_size=224, num_hidden_layers=3,
              num_attention_heads=3, num_key_value_heads=1, vocab_size=384, max_position_embeddings=256,
              rms_norm_eps=1e-5, rope_theta=1000000.0, tie_word_embeddings=False, eos_token_id=[382, 383],
              architectures=["Qwen2ForCausalLM"])
# head size 48 (a step of 16 that is no power of two), 5 heads in 5 groups, long enough for hundreds of keys
TINY_C = dict(model_type="qwen2", hidden_act="silu", hidden_size=240, intermediate_size=176, num_hidden_layers=2,
              num_attention_heads=5, num_key_value_heads=5, vocab_size=331, max_position_embeddings=1024,
              rms_norm_eps=1e-6, rope_theta=50000.0, tie_word_embeddings=True, eos_token_id=0)
PAGE_SIZE = {"A": 16, "B": 8, "C": 16}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C}
SEEDS = {"A": 11, "B": 23, "C": 37}
WEIGHT_STD = 0.08   # wide enough that attention is not near-uniform and logits are of order one

# Bounds of |engine - plain| on logits.  float32: rounding of float32 sums against float64 sums.
# bfloat16: the plain side rounds to bfloat16 at the same places as the engine, so what remains is
# one-unit flips of those roundings (2^-8 relative) carried through the layers.
def tolerance(dtype: str, ref: np.ndarray) -> float:
    scale = max(1.0, float(np.abs(ref).max()))
    return (2e-5 if dtype == "float32" else 3e-2) * scale


def make_model_folder(root: str, name: str, storage=torch.bfloat16) -> str:
    """A model folder of tiny configuration `name`, written by the engine's random-weights mode."""
    import sprout_lm_amd as S
    from sprout_lm_amd.weights import write_model_folder
    folder = os.path.join(root, f"tiny_{name}_{str(storage).split('.')[-1]}")
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        cfg = S.config_from_dict(CONFIGS[name])
        write_model_folder(folder, cfg, SEEDS[name], dtype=storage, std=WEIGHT_STD)
    return folder


_PLAIN_CACHE: dict = {}


def plain_model(folder: str, dtype: str):
    key = (folder, dtype)
    if key not in _PLAIN_CACHE:
        _PLAIN_CACHE[key] = P.load_folder(folder, dtype)
    return _PLAIN_CACHE[key]


_LOGIT_CACHE: dict = {}


def plain_logits(folder: str, dtype: str, tokens, rows=None) -> np.ndarray:
    """Logits of the plain implementation at every position of `tokens`, or at `rows` only (cached per sequence)."""
    key = (folder, dtype, tuple(tokens), None if rows is None else tuple(rows))
    if key not in _LOGIT_CACHE:
        cfg, w = plain_model(folder, dtype)
        store = P.bf16_round if dtype == "bfloat16" else P.f32
        _LOGIT_CACHE[key] = P.forward_logits(w, cfg, list(tokens), store=store, rows=rows)
    return _LOGIT_CACHE[key]


def random_tokens(vocab: int, n: int, seed: int) -> list[int]:
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, n)]
