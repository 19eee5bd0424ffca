"""Configuration of the dense Qwen2 decoder (reference: src/qwen.ts:7-40)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar, Mapping

from .base import ConfigError, ModelConfig, positive_float, positive_int, token_id_list


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    """Every size and constant of a Qwen2 model, as config.json gives them.

    The same keys are required and the same options are refused as in the
    reference's parseQwenConfig (src/qwen.ts:14-34): no key has a default.
    """

    architecture: ClassVar[str] = "Qwen2ForCausalLM"
    model_types: ClassVar[tuple[str, ...]] = ("qwen2",)

    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    vocab_size: int
    max_position_embeddings: int
    rms_norm_eps: float
    rope_theta: float
    tie_word_embeddings: bool
    eos_token_ids: tuple[int, ...]
    hidden_act: str = "silu"

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen2Config":
        if not isinstance(raw, Mapping):
            raise ConfigError("Invalid Qwen2 config: expected a JSON object.")
        # src/qwen.ts:17
        if raw.get("model_type") != "qwen2" or raw.get("hidden_act") != "silu":
            raise ConfigError("Only model_type 'qwen2' with hidden_act 'silu' is supported, got "
                              f"model_type={raw.get('model_type')!r}, hidden_act={raw.get('hidden_act')!r}.")
        # src/qwen.ts:18-20
        refused = [k for k in ("use_sliding_window", "rope_scaling", "quantization_config", "use_mrope") if raw.get(k)]
        if refused:
            raise ConfigError("Sliding window, scaled or multimodal RoPE and quantized checkpoints are not "
                              f"supported (config sets {', '.join(refused)}).")
        ints = {k: positive_int(raw, k) for k in (
            "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
            "num_key_value_heads", "vocab_size", "max_position_embeddings")}
        floats = {k: positive_float(raw, k) for k in ("rms_norm_eps", "rope_theta")}
        tied = raw.get("tie_word_embeddings")
        if not isinstance(tied, bool):
            raise ConfigError("tie_word_embeddings must be boolean.")
        # src/qwen.ts:29-31
        heads, kv_heads, hidden = ints["num_attention_heads"], ints["num_key_value_heads"], ints["hidden_size"]
        if hidden % heads or (hidden // heads) % 2 or heads % kv_heads:
            raise ConfigError(f"Unsupported Qwen2 head dimensions: hidden_size {hidden}, "
                              f"{heads} heads, {kv_heads} key/value heads.")
        if raw.get("head_dim") is not None and raw["head_dim"] != hidden // heads:
            raise ConfigError(f"head_dim {raw['head_dim']} differs from hidden_size / num_attention_heads "
                              f"= {hidden // heads}.")
        eos = token_id_list(raw.get("eos_token_id"), ints["vocab_size"], "eos_token_id")
        return cls(**ints, **floats, tie_word_embeddings=tied, eos_token_ids=eos)

    def to_dict(self) -> dict:
        return {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "hidden_act": self.hidden_act,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "eos_token_id": list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0],
            "use_sliding_window": False,
            "rope_scaling": None,
        }
