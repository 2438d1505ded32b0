from .engine_config import EngineConfig, normalize_dtype, parse_random_weights, preset_names
from .model_config import ConfigError, Qwen3Config, read_config_json

__all__ = ["EngineConfig", "normalize_dtype", "parse_random_weights", "preset_names", "ConfigError", "Qwen3Config", "read_config_json"]
