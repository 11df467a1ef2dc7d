"""Configuration: the engine's, and what every architecture's own configuration shares. Importing this package
imports no torch."""
from .engine import DTYPES, EngineConfig, SamplingParams
from .model import ConfigError, read_config_json

__all__ = ["DTYPES", "EngineConfig", "SamplingParams", "ConfigError", "read_config_json"]
