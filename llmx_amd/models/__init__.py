"""Architectures: name -> configuration class and model assembly."""

from .registry import (ArchitectureEntry, architecture_of, architectures, assemble, read_config, read_model_dir,
                       register_architecture, unregister_architecture)
from . import minimax_m3  # noqa: F401  (registers MiniMaxM3ForCausalLM)

__all__ = ["ArchitectureEntry", "architecture_of", "architectures", "assemble", "read_config", "read_model_dir",
           "register_architecture", "unregister_architecture"]
