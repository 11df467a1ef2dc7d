"""Configuration: the model's (from config.json) and the engine's. Importing this package imports no torch."""
from .engine import DTYPES, EngineConfig, SamplingParams
from .model import ConfigError, Qwen3Config, read_config_json

__all__ = ["DTYPES", "EngineConfig", "SamplingParams", "ConfigError", "Qwen3Config", "read_config_json"]
