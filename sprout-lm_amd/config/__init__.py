from .base import ConfigError, ModelConfig, read_config_json
from .qwen2 import Qwen2Config
from .engine_options import EngineOptions

__all__ = ["ConfigError", "ModelConfig", "read_config_json", "Qwen2Config", "EngineOptions"]
