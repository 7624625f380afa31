"""Typed configurations read from config.json."""

from .reader import ConfigError, KeyReader, read_json
from .minimax_m3 import MiniMaxM3Config

__all__ = ["ConfigError", "KeyReader", "read_json", "MiniMaxM3Config"]
