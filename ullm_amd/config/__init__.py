from .engine_config import EngineConfig, normalize_dtype
from .model_config import ConfigError, Qwen3Config, read_config_json

__all__ = ["EngineConfig", "normalize_dtype", "ConfigError", "Qwen3Config", "read_config_json"]
