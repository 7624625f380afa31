"""Typed, strict reading of a config.json.

Every key that changes the arithmetic must be present and in range; a key the
architecture does not read is refused by name unless it is on the
architecture's list of keys without effect.  The two refusal texts follow the
reference's discipline for model metadata ("missing metadata K" /
"unsupported metadata K": /root/reference/src/model/arch/minimax_m3.hpp:58-63,
typed getters in /root/reference/src/model/arch/metadata.hpp:17-77), spelled
with config.json's own key names.
"""

from __future__ import annotations

import json
import math
from pathlib import Path
from typing import Any, Iterable, Mapping


class ConfigError(ValueError):
    """A config.json the engine refuses; the text names the key."""


_MISSING = object()


class KeyReader:
    """Reads keys of one JSON object and remembers which ones were read."""

    def __init__(self, values: Mapping[str, Any], where: str = "config.json"):
        if not isinstance(values, Mapping):
            raise ConfigError(f"config: {where} is not a JSON object")
        self._values = values
        self._where = where
        self._read: set[str] = set()

    # -- refusals -----------------------------------------------------------
    def missing(self, key: str) -> ConfigError:
        return ConfigError(f"config: missing key {self._path(key)}")

    def unsupported(self, key: str, why: str = "") -> ConfigError:
        tail = f" ({why})" if why else ""
        return ConfigError(f"config: unsupported value for {self._path(key)}{tail}")

    def _path(self, key: str) -> str:
        return key if self._where == "config.json" else f"{self._where}.{key}"

    # -- raw access -----------------------------------------------------------
    def has(self, key: str) -> bool:
        return key in self._values and self._values[key] is not None

    def raw(self, key: str, default: Any = _MISSING) -> Any:
        self._read.add(key)
        if not self.has(key):
            if default is _MISSING:
                raise self.missing(key)
            return default
        return self._values[key]

    # -- typed getters ----------------------------------------------------
    def integer(self, key: str, lo: int = 1, hi: int = 2**31 - 1, default: Any = _MISSING) -> int:
        v = self.raw(key, default)
        if v is default and default is not _MISSING:
            return v
        if isinstance(v, bool) or not isinstance(v, (int, float)) or v != int(v):
            raise self.unsupported(key, f"{v!r} is not a whole number")
        v = int(v)
        if not lo <= v <= hi:
            raise self.unsupported(key, f"{v} is outside [{lo}, {hi}]")
        return v

    def real(self, key: str, lo: float = -math.inf, hi: float = math.inf, default: Any = _MISSING,
             positive: bool = False) -> float:
        v = self.raw(key, default)
        if v is default and default is not _MISSING:
            return v
        if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v):
            raise self.unsupported(key, f"{v!r} is not a finite number")
        v = float(v)
        if not lo <= v <= hi or (positive and v <= 0.0):
            raise self.unsupported(key, f"{v} is out of range")
        return v

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self.raw(key, default)
        if v is default and default is not _MISSING:
            return v
        if not isinstance(v, bool):
            raise self.unsupported(key, f"{v!r} is not true or false")
        return v

    def choice(self, key: str, allowed: Iterable[Any], default: Any = _MISSING) -> Any:
        v = self.raw(key, default)
        allowed = list(allowed)
        if v not in allowed:
            raise self.unsupported(key, f"{v!r}; this engine computes {allowed}")
        return v

    def held(self, key: str, value: Any) -> None:
        """An optional key that, when present, may only hold `value`."""
        if self.has(key):
            v = self.raw(key)
            if v != value:
                raise self.unsupported(key, f"{v!r}; this engine computes only {value!r}")
        else:
            self._read.add(key)

    def child(self, key: str, required: bool = True) -> "KeyReader | None":
        if not self.has(key):
            self._read.add(key)
            if required:
                raise self.missing(key)
            return None
        return KeyReader(self.raw(key), where=self._path(key))

    # -- closing ----------------------------------------------------------
    def finish(self, without_effect: Iterable[str], architecture: str) -> None:
        """Refuse, by name, every key that was neither read nor listed as having no effect."""
        ignored = set(without_effect)
        for key in self._values:
            if key not in self._read and key not in ignored:
                raise ConfigError(
                    f"config: key {self._path(key)} is not one this engine reads for {architecture}")


def read_json(path: str | Path) -> dict:
    path = Path(path)
    try:
        with open(path, "r", encoding="utf-8") as f:
            return json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"config: {path} does not exist") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"config: {path} is not valid JSON: {e}") from None
