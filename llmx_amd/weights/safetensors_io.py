"""A strict safetensors reader and a writer.

The container: an 8-byte little-endian header length, a JSON header whose
entries hold exactly `dtype`, `shape` and `data_offsets`, then the data area.
The reader keeps the reference's rules (/root/reference/src/format/safetensors.hpp:
dtype map :52-64, entry rules :66-86, file rules :107-130): no key twice in the
header or in an entry, `__metadata__` an object of strings, offsets span the
shape, tensors tile the data area without gap or overlap, each at a file offset
aligned to its element (at most to 4 bytes), and end at the file's end.  Tensors are returned as torch views over a memory map, so a large file
is never read whole.
"""

from __future__ import annotations

import json
import mmap
import struct
from dataclasses import dataclass
from pathlib import Path
from typing import Dict, Iterable, Mapping, Tuple

import torch

MAX_HEADER_BYTES = 100 << 20

DTYPES = {
    "F32": (torch.float32, 4),
    "F16": (torch.float16, 2),
    "BF16": (torch.bfloat16, 2),
    "I32": (torch.int32, 4),
    "I64": (torch.int64, 8),
}
NAMES = {v[0]: k for k, v in DTYPES.items()}


class SafetensorsError(ValueError):
    pass


def parse_json_unique(text: str, what: str):
    """json.loads that refuses an object that holds a key twice (the standard parser silently keeps the last one;
    the reference refuses: /root/reference/src/format/safetensors.hpp:40-44,109)."""
    def pairs(items):
        seen = {}
        for k, v in items:
            if k in seen:
                raise SafetensorsError(f"{what} repeats key {k}")
            seen[k] = v
        return seen
    return json.loads(text, object_pairs_hook=pairs)


@dataclass(frozen=True)
class TensorEntry:
    name: str
    dtype: torch.dtype
    shape: Tuple[int, ...]
    begin: int  # byte offsets in the data area
    end: int


class SafetensorsFile:
    """An open file: its entries by name, and each tensor as a view over the map."""

    def __init__(self, path: str | Path):
        self.path = Path(path)
        try:
            self._file = open(self.path, "rb")
        except FileNotFoundError:
            raise SafetensorsError(f"safetensors: {self.path} does not exist") from None
        size = self.path.stat().st_size
        if size < 8:
            raise SafetensorsError(f"safetensors: {self.path} is shorter than its header length")
        (n,) = struct.unpack("<Q", self._file.read(8))
        if n > MAX_HEADER_BYTES or 8 + n > size:
            raise SafetensorsError(f"safetensors: {self.path} declares a header of {n} bytes, beyond the file or the limit")
        try:
            header = parse_json_unique(self._file.read(n).decode("utf-8"), f"safetensors header of {self.path}")
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise SafetensorsError(f"safetensors: {self.path} header is not JSON: {e}") from None
        if not isinstance(header, dict):
            raise SafetensorsError(f"safetensors: {self.path} header is not an object")
        self.metadata = header.pop("__metadata__", {})
        if not isinstance(self.metadata, dict):
            raise SafetensorsError(f"safetensors: __metadata__ of {self.path} is not an object")
        for k, v in self.metadata.items():
            if not isinstance(v, str):
                raise SafetensorsError(f"safetensors: __metadata__ value of {k} in {self.path} is not a string")
        self.data_start = 8 + n
        data_bytes = size - self.data_start
        self.entries: Dict[str, TensorEntry] = {}
        for name, e in header.items():
            if not isinstance(e, dict) or set(e) != {"dtype", "shape", "data_offsets"}:
                raise SafetensorsError(f"safetensors tensor {name} must hold exactly dtype, shape and data_offsets")
            if e["dtype"] not in DTYPES:
                raise SafetensorsError(f"safetensors tensor {name} has dtype {e['dtype']}, which this engine does not read")
            dtype, width = DTYPES[e["dtype"]]
            shape = e["shape"]
            if not isinstance(shape, list) or len(shape) > 5 or any(not isinstance(d, int) or isinstance(d, bool) or d < 0 for d in shape):
                raise SafetensorsError(f"safetensors tensor {name} has an invalid shape {shape!r}")
            off = e["data_offsets"]
            if not isinstance(off, list) or len(off) != 2 or any(not isinstance(o, int) or isinstance(o, bool) for o in off):
                raise SafetensorsError(f"safetensors tensor {name} has invalid data_offsets {off!r}")
            count = 1
            for d in shape:
                count *= d
            if off[0] < 0 or off[1] - off[0] != count * width or off[1] > data_bytes:
                raise SafetensorsError(f"safetensors tensor {name}: data_offsets {off} do not span its shape {shape} of {e['dtype']}")
            self.entries[name] = TensorEntry(name, dtype, tuple(shape), off[0], off[1])
        at = 0
        for e in sorted(self.entries.values(), key=lambda t: (t.begin, t.end)):
            if e.begin != at:
                raise SafetensorsError(f"safetensors: {self.path} has a gap or an overlap before tensor {e.name}")
            align = min(4, DTYPES[NAMES[e.dtype]][1])
            if (self.data_start + e.begin) % align:
                raise SafetensorsError(f"safetensors tensor {e.name} is not at a {align}-byte-aligned file offset in {self.path}")
            at = e.end
        if at != data_bytes:
            raise SafetensorsError(f"safetensors: {self.path} does not end where its last tensor ends")
        self._map = mmap.mmap(self._file.fileno(), 0, access=mmap.ACCESS_READ) if size else None

    def names(self) -> Iterable[str]:
        return self.entries.keys()

    def tensor(self, name: str) -> torch.Tensor:
        """A read-only CPU view of the tensor's bytes in the map (copy it before writing to it)."""
        e = self.entries[name]
        count = 1
        for d in e.shape:
            count *= d
        if count == 0:
            return torch.empty(e.shape, dtype=e.dtype)
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")  # torch warns that the buffer is not writable; it is never written
            flat = torch.frombuffer(self._map, dtype=e.dtype, count=count, offset=self.data_start + e.begin)
        return flat.view(e.shape)

    def close(self) -> None:
        # views handed out keep the map alive; closing is left to the collector when any exist
        try:
            if self._map is not None:
                self._map.close()
        except BufferError:
            pass
        self._file.close()


def write_safetensors(path: str | Path, tensors: Mapping[str, torch.Tensor], metadata: Mapping[str, str] | None = None) -> None:
    """Writes CPU tensors, each contiguous, the data area aligned to 8 bytes; wider elements first (in the order given
    among equals), so that every tensor lies at an offset aligned to its element."""
    header = {}
    if metadata:
        header["__metadata__"] = dict(metadata)
    at = 0
    ordered = sorted(tensors.items(), key=lambda item: -item[1].element_size())
    for name, t in ordered:
        if t.dtype not in NAMES:
            raise SafetensorsError(f"safetensors: tensor {name} has dtype {t.dtype}, which the writer does not write")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [at, at + nbytes]}
        at += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name, t in ordered:
            t = t.detach().cpu().contiguous()
            if t.numel():
                f.write(t.view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes())
