"""Qwen2 as a plan of parts (reference: QwenRunner, src/qwen.ts:95-204; tensor names :135-153)."""
from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from .plan import LayerCall, LayerPlan, ModelPlan, PartPlan


def build_qwen2(cfg: Qwen2Config) -> ModelPlan:
    H, hd = cfg.hidden_size, cfg.head_dim
    layers = []
    for i in range(cfg.num_hidden_layers):
        base = f"model.layers.{i}."
        rotary = PartPlan("position", "rotary_neox", {"head_dim": hd, "theta": cfg.rope_theta})
        layers.append(LayerPlan("pre_norm", {
            "mixer_norm": PartPlan("norm", "rmsnorm", {"size": H, "eps": cfg.rms_norm_eps}, base + "input_layernorm."),
            "mixer": PartPlan("mixer", "attention", {
                "hidden": H, "heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": hd,
                "position": rotary, "qkv_bias": True, "out_bias": False, "window": None}, base + "self_attn."),
            "ffn_norm": PartPlan("norm", "rmsnorm", {"size": H, "eps": cfg.rms_norm_eps},
                                 base + "post_attention_layernorm."),
            "ffn": PartPlan("feed_forward", "gated_mlp", {"hidden": H, "inner": cfg.intermediate_size,
                                                          "activation": cfg.hidden_act}, base + "mlp."),
        }))
    return ModelPlan(
        architecture=cfg.architecture, config=cfg, hidden_size=H, vocab_size=cfg.vocab_size,
        max_positions=cfg.max_position_embeddings, eos_token_ids=cfg.eos_token_ids,
        embedding=PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab_size, "hidden": H}, "model.embed_tokens."),
        layers=layers,
        schedule=[LayerCall(i, i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartPlan("norm", "rmsnorm", {"size": H, "eps": cfg.rms_norm_eps}, "model.norm."),
        head=PartPlan("head", "linear_head", {"vocab": cfg.vocab_size, "hidden": H, "tied": cfg.tie_word_embeddings},
                      "lm_head."),
        # a tied checkpoint may still ship the output matrix (reference reads only what it asks for,
        # src/safetensors.ts:79-81)
        ignorable_tensors=frozenset({"lm_head.weight"} if cfg.tie_word_embeddings else ()),
    )
