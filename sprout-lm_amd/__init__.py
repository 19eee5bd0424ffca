"""A single-GPU inference engine for AMD MI355X: everything between a request's token ids and its
next token, put together from parts, with hand-written HIP kernels."""
from .config import ConfigError, EngineOptions, ModelConfig, Qwen2Config
from .registry import (build_model_plan, config_from_dict, load_config, register_architecture,
                       registered_architectures)

__version__ = "0.1.0"
__all__ = ["ConfigError", "EngineOptions", "ModelConfig", "Qwen2Config", "build_model_plan", "config_from_dict",
           "load_config", "register_architecture", "registered_architectures"]
