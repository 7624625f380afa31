"""Weights by tensor name: check everything against the model's list first, then bring each tensor to the device.

The file's tensors must be exactly the ones the model's parts name, each with the shape its part expects; otherwise
one error lists every missing tensor, every unexpected tensor and every wrong shape, and nothing is loaded
(the reference validates headers and the plan before any byte streams: /root/reference/src/inference/load.hpp:316-422,
/root/reference/src/model/runtime.hpp:582-653).

Types on the device: matrices and tables stay bfloat16 when stored so (a tensor stored in 32 bits stays 32 bits; half
precision is widened to 32 bits); the 32-bit path widens everything to float32, which is exact.  Norm weights, biases
and router matrices are float32 in both paths.  Integer tables are int32.
"""

from __future__ import annotations

import json
from pathlib import Path
from typing import Dict, Iterable, List, Tuple

import torch

from ..parts.spec import TensorSpec
from .safetensors_io import SafetensorsError, SafetensorsFile, parse_json_unique


class WeightsError(ValueError):
    """Weights that do not fit the model; `missing`, `unexpected` and `wrong_shape` hold the details."""

    def __init__(self, text, missing=(), unexpected=(), wrong_shape=(), wrong_type=()):
        super().__init__(text)
        self.missing = list(missing)
        self.unexpected = list(unexpected)
        self.wrong_shape = list(wrong_shape)
        self.wrong_type = list(wrong_type)


class ModelFiles:
    """The safetensors files of a model folder as one name -> tensor source."""

    def __init__(self, folder: str | Path):
        folder = Path(folder)
        index = folder / "model.safetensors.index.json"
        single = folder / "model.safetensors"
        if index.exists():
            try:
                root = parse_json_unique(index.read_text(), f"safetensors index {index}")
            except json.JSONDecodeError as e:
                raise WeightsError(f"weights: {index} is not JSON: {e}") from None
            weight_map = root.get("weight_map") if isinstance(root, dict) else None
            if not isinstance(weight_map, dict):
                raise WeightsError(f"weights: {index} has no weight_map object")
            for tensor, file_name in weight_map.items():
                if not isinstance(file_name, str):
                    raise WeightsError(f"weights: {index}: the weight_map value of {tensor} is not a file name")
                # a file named by an index sits beside it (/root/reference/src/format/safetensors.hpp:134-137)
                if file_name in ("", ".", "..") or any(c in file_name for c in "/\\:"):
                    raise WeightsError(f"weights: {index} names a file outside its directory: {file_name}")
            names = sorted(set(weight_map.values()))
            self.files = [SafetensorsFile(folder / n) for n in names]
            held = {t for f in self.files for t in f.names()}
            if held != set(weight_map):
                raise WeightsError(f"weights: {index} does not name exactly the tensors its files hold",
                                   missing=sorted(set(weight_map) - held), unexpected=sorted(held - set(weight_map)))
        elif single.exists():
            self.files = [SafetensorsFile(single)]
        else:
            shards = sorted(folder.glob("*.safetensors"))
            if not shards:
                raise WeightsError(f"weights: {folder} holds no model.safetensors")
            self.files = [SafetensorsFile(p) for p in shards]
        self.where: Dict[str, SafetensorsFile] = {}
        for f in self.files:
            for n in f.names():
                if n in self.where:
                    raise WeightsError(f"weights: duplicate tensor {n}")
                self.where[n] = f

    def names(self) -> Iterable[str]:
        return self.where.keys()

    def entry(self, name: str):
        return self.where[name].entries[name]

    def tensor(self, name: str) -> torch.Tensor:
        return self.where[name].tensor(name)

    def close(self) -> None:
        for f in self.files:
            f.close()


_FLOATS = (torch.float32, torch.bfloat16, torch.float16)
_INTS = (torch.int32, torch.int64)


def device_dtype(spec: TensorSpec, stored: torch.dtype, exact: bool) -> torch.dtype:
    """The type a tensor has on the device: what its spec states, else what its role says."""
    if spec.dtype is not None:
        return getattr(torch, spec.dtype)
    if spec.role == "int":
        return torch.int32
    if spec.role in ("norm", "bias", "router") or exact:
        return torch.float32
    return torch.bfloat16 if stored == torch.bfloat16 else torch.float32


def _wants_ints(spec: TensorSpec) -> bool:
    return spec.dtype == "int32" if spec.dtype is not None else spec.role == "int"


def check(specs: List[TensorSpec], held: Dict[str, Tuple[torch.dtype, Tuple[int, ...]]], exact: bool = False) -> None:
    """Raises one WeightsError naming every tensor that is missing, unexpected, of a wrong shape or of a wrong type,
    and every fused target whose slices (`TensorSpec.into`) would arrive in different device types."""
    wanted = {s.name: s for s in specs}
    if len(wanted) != len(specs):
        seen, twice = set(), []
        for s in specs:
            if s.name in seen:
                twice.append(s.name)
            seen.add(s.name)
        raise WeightsError(f"weights: the model names a tensor twice: {twice}")
    missing = sorted(n for n in wanted if n not in held)
    unexpected = sorted(n for n in held if n not in wanted)
    wrong_shape, wrong_type = [], []
    for n, s in wanted.items():
        if n not in held:
            continue
        dtype, shape = held[n]
        if tuple(shape) != tuple(s.shape):
            wrong_shape.append((n, tuple(shape), tuple(s.shape)))
        if dtype not in (_INTS if _wants_ints(s) else _FLOATS):
            wrong_type.append((n, str(dtype)))
    # the slices of one fused tensor must agree in their device type: found here, before anything is allocated
    fused: Dict[str, Dict[str, List[str]]] = {}
    for n, s in wanted.items():
        if s.into is not None and n in held:
            fused.setdefault(s.into[0], {}).setdefault(str(device_dtype(s, held[n][0], exact)), []).append(n)
    mixed = {target: kinds for target, kinds in fused.items() if len(kinds) > 1}
    if missing or unexpected or wrong_shape or wrong_type or mixed:
        lines = ["weights: the file's tensors are not the model's"]
        if missing:
            lines.append(f"  missing ({len(missing)}): " + ", ".join(missing))
        if unexpected:
            lines.append(f"  unexpected ({len(unexpected)}): " + ", ".join(unexpected))
        for n, got, want in wrong_shape:
            lines.append(f"  wrong shape: {n} is {list(got)}, expected {list(want)}")
        for n, t in wrong_type:
            lines.append(f"  wrong type: {n} is stored as {t}")
        for target, kinds in sorted(mixed.items()):
            lines.append(f"  mixed types: the parts of {target} are stored in different types: "
                         + "; ".join(f"{len(names)} as {kind} (first: {sorted(names)[0]})" for kind, names in sorted(kinds.items())))
            wrong_type.extend((n, kind) for kind, names in kinds.items() for n in names)
        raise WeightsError("\n".join(lines), missing, unexpected, wrong_shape, wrong_type)


def load(specs: List[TensorSpec], files: ModelFiles, device: torch.device, exact: bool) -> Dict[str, torch.Tensor]:
    check(specs, {n: (files.entry(n).dtype, files.entry(n).shape) for n in files.names()}, exact)
    out: Dict[str, torch.Tensor] = {}
    for s in specs:
        host = files.tensor(s.name)
        dtype = device_dtype(s, host.dtype, exact)
        if s.into is None:
            out[s.name] = host.to(device=device, dtype=dtype).contiguous()
            continue
        target, shape, index = s.into
        if target not in out:
            out[target] = torch.empty(shape, dtype=dtype, device=device)
        out[target][index].copy_(host.to(dtype))
    return out
