from .engine_config import EngineConfig, normalize_dtype, parse_random_weights, preset_names
from .model_config import ConfigError, DovisunConfig, KumudraConfig, PamopelConfig, Qwen3Config, ZiferaxConfig, read_config_json

__all__ = ["EngineConfig", "normalize_dtype", "parse_random_weights", "preset_names", "ConfigError", "DovisunConfig", "KumudraConfig", "PamopelConfig", "Qwen3Config", "ZiferaxConfig", "read_config_json"]
