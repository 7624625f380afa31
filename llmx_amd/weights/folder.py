"""The random-weights mode: a model folder (config.json, model.safetensors) from a configuration and a seed."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from ..parts.base import BuildContext
from .random_init import RandomInit, host_values, stored_dtype
from .safetensors_io import write_safetensors


def model_tensor_specs(config):
    """The tensors the configuration's model reads (built on the CPU: only names and shapes are needed)."""
    from ..engine.model import BuiltModel
    from ..models import registry
    spec = registry.assemble(config)
    model = BuiltModel(spec, BuildContext(torch.float32, torch.device("cpu"), 1))
    return model.tensor_specs()


def random_tensors(config, init: RandomInit) -> dict:
    """name -> CPU tensor in its stored type."""
    out = {}
    for s in model_tensor_specs(config):
        out[s.name] = host_values(s, init).to(stored_dtype(s, init))
    return out


def write_random_model(folder: str | Path, config, init: RandomInit = RandomInit()) -> Path:
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(config.to_json(), indent=2) + "\n")
    write_safetensors(folder / "model.safetensors", random_tensors(config, init),
                      metadata={"format": "pt", "seed": str(init.seed)})
    return folder
