"""What a step reads and computes, summed over a model's parts, against the closed formulas of the sizes.

W_layer = H(Q+2KV) + (Q+2KV) + QH + 3HI + 2H;  W_step = L W_layer + VH + H (the output matrix is read whether
tied or not);  KV bytes = B ctx 2 L KV size;  F_prefill = 2T L (H(Q+2KV) + QH + 3HI) + 2 L Q T^2 + 2VH."""
import pytest

import sprout_lm_amd as S
from sprout_lm_amd.cli import PRESETS

WANT = {"qwen2.5-0.5b": (0.988, 1.65), "qwen2.5-7b": (14.14, 27.6), "qwen2.5-32b": (63.97, 130.6)}   # GB a step, TF a prefill


@pytest.mark.parametrize("name", sorted(WANT))
def test_parts_add_up_to_the_formulas(name):
    raw = PRESETS[name]
    parts = S.build_model_plan(S.config_from_dict(raw)).instantiate()
    H, I, L, V = raw["hidden_size"], raw["intermediate_size"], raw["num_hidden_layers"], raw["vocab_size"]
    hd = H // raw["num_attention_heads"]
    Q, KV = H, raw["num_key_value_heads"] * hd
    layer = H * (Q + 2 * KV) + (Q + 2 * KV) + Q * H + 3 * H * I + 2 * H
    step = L * layer + V * H + H
    assert parts.weight_bytes(2) == 2 * step and parts.weight_bytes(4) == 4 * step
    assert abs(2 * step / 1e9 - WANT[name][0]) < 0.01
    for batch, context in ((1, 512), (8, 4096), (64, 512)):
        assert batch * context * parts.cache_bytes_per_context_token(2) == batch * context * 2 * L * KV * 2
    T = 2048
    flops = 2.0 * T * L * (H * (Q + 2 * KV) + Q * H + 3 * H * I) + 2.0 * L * Q * T * T + 2.0 * V * H
    assert parts.flops(T, T * T // 2, 1) == pytest.approx(flops, rel=1e-12)
    assert abs(flops / 1e12 - WANT[name][1]) < 0.06
    # one decoded token at a context of 100: the projections once, 100 pairs in every layer, one row of logits
    one = 2.0 * L * (H * (Q + 2 * KV) + Q * H + 3 * H * I) + 4.0 * L * Q * 100 + 2.0 * V * H
    assert parts.flops(1, 100, 1) == pytest.approx(one, rel=1e-12)


def test_a_layer_that_runs_twice_reads_its_weights_once():
    from sprout_lm_amd.models.plan import LayerCall
    raw = dict(PRESETS["tiny-a"])
    once = S.build_model_plan(S.config_from_dict(raw)).instantiate()
    plan = S.build_model_plan(S.config_from_dict(raw))
    plan.schedule = plan.schedule + [LayerCall(0, 2)]       # layer 0 again, with a cache slot of its own
    twice = plan.instantiate()
    assert twice.weight_bytes(2) == once.weight_bytes(2)
    assert twice.cache_bytes_per_context_token(2) == once.cache_bytes_per_context_token(2) * 3 // 2
    assert twice.flops(5, 15, 1) > once.flops(5, 15, 1)
