"""Configuration and registry (reference: parseQwenConfig, src/qwen.ts:14-34; test/qwen.test.ts:94-100)."""
import json

import pytest

import sprout_lm_amd as S
from sprout_lm_amd.config import ConfigError, EngineOptions, Qwen2Config
from tests import helpers as H


def test_qwen2_config_reads_its_own_keys():
    cfg = S.config_from_dict(H.TINY_B)
    assert isinstance(cfg, Qwen2Config)
    assert (cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (96, 3, 1, 32)
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 1e6 and cfg.tie_word_embeddings is False
    assert cfg.eos_token_ids == (382, 383)
    again = S.config_from_dict(cfg.to_dict())
    assert again == cfg


def test_architecture_is_chosen_by_config_json():
    assert S.config_from_dict(H.TINY_A).architecture == "Qwen2ForCausalLM"        # by model_type
    assert S.config_from_dict(dict(H.TINY_A, architectures=None)).architecture == "Qwen2ForCausalLM"
    with pytest.raises(ConfigError, match="registered"):
        S.config_from_dict(dict(H.TINY_A, architectures=["LlamaForCausalLM"]))
    with pytest.raises(ConfigError, match="registered"):
        S.config_from_dict({"model_type": "gpt2"})


@pytest.mark.parametrize("change", [
    {"model_type": "llama"}, {"hidden_act": "gelu"}, {"rope_scaling": {"type": "linear"}}, {"use_sliding_window": True},
    {"quantization_config": {"bits": 4}}, {"use_mrope": True}, {"num_key_value_heads": 3}, {"rms_norm_eps": 0},
    {"rope_theta": -1.0}, {"eos_token_id": -1}, {"eos_token_id": 256}, {"hidden_size": 66}, {"head_dim": 8},
    {"tie_word_embeddings": "yes"}, {"vocab_size": 0}, {"num_hidden_layers": 2.5}, {"hidden_size": True},
])
def test_unsupported_configurations_fail_before_weights_load(change):
    raw = dict(H.TINY_A, architectures=["Qwen2ForCausalLM"], **change)
    with pytest.raises(ConfigError):
        S.config_from_dict(raw)


@pytest.mark.parametrize("key", ["hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                                 "num_key_value_heads", "vocab_size", "max_position_embeddings", "rms_norm_eps",
                                 "rope_theta", "tie_word_embeddings", "eos_token_id"])
def test_no_size_or_constant_has_a_default(key):
    raw = {k: v for k, v in H.TINY_A.items() if k != key}
    with pytest.raises(ConfigError):
        S.config_from_dict(raw)


def test_head_dim_is_accepted_when_consistent():
    assert S.config_from_dict(dict(H.TINY_A, head_dim=16)).head_dim == 16


def test_plan_sizes_follow_the_config():
    plan = S.build_model_plan(S.config_from_dict(H.TINY_B))
    expected = plan.expected_tensors()
    assert expected["model.layers.2.self_attn.k_proj.weight"].shape == (32, 96)
    assert expected["model.layers.0.self_attn.q_proj.bias"].shape == (96,)
    assert expected["model.layers.1.mlp.down_proj.weight"].shape == (96, 224)
    assert expected["lm_head.weight"].shape == (384, 96)
    assert "lm_head.weight" not in S.build_model_plan(S.config_from_dict(H.TINY_A)).expected_tensors()
    assert len(plan.schedule) == 3 and [c.cache_slot for c in plan.schedule] == [0, 1, 2]


def test_engine_options_are_positive_integers_or_booleans():
    assert EngineOptions().block_size == 16
    for bad in ({"block_size": 0}, {"max_batch_tokens": float("nan")}, {"num_blocks": -1}, {"prefix_caching": 1},
                {"max_sequences": True}):
        with pytest.raises(ConfigError):
            EngineOptions(**bad)


def test_load_config_from_folder(tmp_path):
    (tmp_path / "config.json").write_text(json.dumps(H.TINY_A))
    assert S.load_config(str(tmp_path)).vocab_size == 256
    with pytest.raises(ConfigError):
        S.load_config(str(tmp_path / "missing"))


def test_sizes_that_no_kernel_takes_are_refused_when_the_parts_are_built():
    """Not at the first step: a head size beyond what the attention kernels take, or a feed-forward activation
    or a rotation pairing without a kernel, fail where the model is put together from config.json."""
    from sprout_lm_amd.config.base import ConfigError
    from sprout_lm_amd.models.plan import PartPlan
    from sprout_lm_amd import ops
    raw = dict(H.TINY_A, hidden_size=1024, num_attention_heads=2, num_key_value_heads=1)     # head size 512: taken
    S.build_model_plan(S.config_from_dict(raw)).instantiate()
    raw = dict(H.TINY_A, hidden_size=1056, num_attention_heads=2, num_key_value_heads=1)     # head size 528
    with pytest.raises(ConfigError, match="head size 528 is outside 1..512"):
        S.build_model_plan(S.config_from_dict(raw)).instantiate()
    with pytest.raises(ValueError, match="'gelu' has no kernel"):
        PartPlan("feed_forward", "gated_mlp", {"hidden": 8, "inner": 8, "activation": "gelu"}).make()
    with pytest.raises(ops.KernelError, match="rotation pairing 'interleaved'"):
        ops.kernels.variant_code(ops.ROTARY_PAIRINGS, "interleaved", "rotation pairing")
    assert ops.ROTARY_PAIRINGS == {"halves": 0} and ops.GATE_ACTIVATIONS == {"silu": 0}
    with pytest.raises(ConfigError, match="score stage 'soft_cap'"):
        PartPlan("mixer", "attention", {"hidden": 32, "heads": 2, "kv_heads": 1, "head_dim": 16, "scores": "soft_cap",
                                        "position": PartPlan("position", "none", {"head_dim": 16})}).make()
    assert ops.SCORE_STAGES == {"scaled_dot": 0}
