"""Device memory is counted before it is taken (reference: native/cuda-offload.cu:249-252)."""
import pytest
import torch

import sprout_lm_amd as S
from sprout_lm_amd.cache import CacheManager, PagedKVSpec, StateSpec
from sprout_lm_amd.cli import PRESETS
from sprout_lm_amd.engine.memory import MIB, MemoryBudget, MemoryBudgetError, check_budget, weight_bytes


def test_weight_bytes_follow_the_formula_of_the_sizes():
    """W_layer = H(Q+2KV) + (Q+2KV) + QH + 3HI + 2H; W = L W_layer + VH + H (+ VH for a separate head)."""
    for name, want_gb in (("qwen2.5-0.5b", 0.988), ("qwen2.5-7b", 15.23), ("qwen2.5-32b", 65.53)):
        raw = PRESETS[name]
        cfg = S.config_from_dict(raw)
        H, I, L, V = raw["hidden_size"], raw["intermediate_size"], raw["num_hidden_layers"], raw["vocab_size"]
        hd = H // raw["num_attention_heads"]
        Q, KV = H, raw["num_key_value_heads"] * hd
        layer = H * (Q + 2 * KV) + (Q + 2 * KV) + Q * H + 3 * H * I + 2 * H
        total = L * layer + V * H + H + (0 if raw["tie_word_embeddings"] else V * H)
        expected = S.build_model_plan(cfg).expected_tensors()
        assert weight_bytes(expected, torch.bfloat16) == 2 * total
        assert weight_bytes(expected, torch.float32) == 4 * total
        assert abs(2 * total / 1e9 - want_gb) < 0.01, (name, 2 * total / 1e9)
        # a checkpoint that stores its norms in 32-bit keeps them so under bfloat16 compute
        stored = {n: (torch.float32 if "norm" in n else torch.bfloat16) for n in expected}
        norms = (2 * L + 1) * H
        assert weight_bytes(expected, torch.bfloat16, stored) == 2 * total + 2 * norms


def test_pool_bytes_count_every_group_and_state():
    cache = CacheManager([PagedKVSpec(2, 64), PagedKVSpec(2, 64), PagedKVSpec(1, 32, window=8), StateSpec((5, 3))],
                         block_size=16, num_blocks=10, max_sequences=4, prefix_caching=False)
    paged = 2 * 2 * 10 * 2 * 16 * 64 + 2 * 1 * 10 * 1 * 16 * 32
    assert cache.storage_bytes(2) == 2 * paged + (4 + 1) * 15 * 4
    assert cache.storage_bytes(4) == 4 * paged + (4 + 1) * 15 * 4


def test_budget_refuses_with_the_three_numbers():
    budget = MemoryBudget(weight_limit_mib=0, reserve_mib=1024)
    check_budget(10 * 1024 * MIB, 5 * 1024 * MIB, 16 * 1024 * MIB, budget)           # 10 + 5 + 1 = 16: fits exactly
    with pytest.raises(MemoryBudgetError) as info:
        check_budget(10 * 1024 * MIB, 5 * 1024 * MIB + 1, 16 * 1024 * MIB, budget)
    text = str(info.value)
    assert "weights 10,240 MiB" in text and "cache pools 5,120 MiB" in text and "reserve 1,024 MiB" in text
    assert "free 16,384 MiB" in text
    with pytest.raises(MemoryBudgetError, match="Resident weight budget exceeded.*limit is 100 MiB"):
        check_budget(101 * MIB, 0, 1 << 40, MemoryBudget(weight_limit_mib=100))
    check_budget(100 * MIB, 0, 1 << 40, MemoryBudget(weight_limit_mib=100))
    with pytest.raises(ValueError):
        MemoryBudget(reserve_mib=-1)
