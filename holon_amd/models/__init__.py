"""Architectures. Importing this package registers them by their config.json name."""
from . import qwen3

__all__ = ["qwen3"]
