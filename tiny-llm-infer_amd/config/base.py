"""Architecture-neutral descriptions of a model: what the typed, per-architecture
configuration is turned into before anything is built.

A ``ModelSpec`` is pure data.  It names the parts of every block (mixer,
feed-forward, norms, position encoding) with their sizes and constants, the
tensor names their weights are stored under, and the order in which blocks run.
Parts are built from it by ``parts.build``; none of them learns which
architecture it belongs to.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Tuple


class ConfigError(ValueError):
    """A config.json is missing a key, holds a value of the wrong type, or
    asks for something this engine does not implement."""


@dataclass(frozen=True)
class PartSpec:
    """One part of a layer: ``kind`` selects the implementation from the part
    registry, ``params`` are its sizes and constants, ``names`` maps the roles
    of its weights to full tensor names in the checkpoint."""
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)
    names: Dict[str, str] = field(default_factory=dict)
    # nested parts (a mixer's position encoding, its inner norms)
    parts: Dict[str, "PartSpec"] = field(default_factory=dict)


@dataclass(frozen=True)
class BlockSpec:
    """A residual block: which arrangement of norm/mixer/feed-forward it uses
    and the parts themselves.  ``ffn`` None: a block of a mixer alone (its arrangement has
    to know what to do without one; "prenorm" then is norm, mixer, sum)."""
    arrangement: str
    mixer: PartSpec
    ffn: Optional[PartSpec]
    norms: Dict[str, PartSpec]


@dataclass(frozen=True)
class LayerCall:
    """One entry of the run order.  ``block`` indexes ``ModelSpec.blocks`` (a
    block may be named by several calls), ``cache`` is the cache layer this
    call's mixer uses (-1: none).  With ``writes_cache`` false the mixer only
    reads that cache layer, which another call has written earlier in the same
    step (shared keys and values)."""
    block: int
    cache: int = -1
    writes_cache: bool = True


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    embedding: PartSpec
    blocks: Tuple[BlockSpec, ...]
    schedule: Tuple[LayerCall, ...]
    final_norm: PartSpec
    head: PartSpec
    eos_token_ids: Tuple[int, ...] = ()

    def num_cache_layers(self) -> int:
        return 1 + max((c.cache for c in self.schedule), default=-1)


# --------------------------------------------------------------------------
# helpers for typed readers of config.json
# --------------------------------------------------------------------------

_MISSING = object()


class JsonReader:
    """Typed access to the keys of one config.json, remembering which keys
    were looked at so that a reader can report what it ignored."""

    def __init__(self, data: Dict[str, Any], origin: str = "config.json"):
        if not isinstance(data, dict):
            raise ConfigError(f"{origin}: top level must be a JSON object")
        self.data = data
        self.origin = origin
        self.seen = set()

    def _get(self, key: str, default: Any = _MISSING) -> Any:
        self.seen.add(key)
        if key not in self.data or self.data[key] is None:
            if default is _MISSING:
                raise ConfigError(f"{self.origin}: required key '{key}' is missing")
            return default
        return self.data[key]

    def raw(self, key: str, default: Any = None) -> Any:
        self.seen.add(key)
        return self.data.get(key, default)

    def integer(self, key: str, default: Any = _MISSING, minimum: Optional[int] = None) -> Any:
        v = self._get(key, default)
        if v is None:
            return None
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                v = int(v)
            else:
                raise ConfigError(f"{self.origin}: '{key}' must be an integer, got {v!r}")
        if minimum is not None and v < minimum:
            raise ConfigError(f"{self.origin}: '{key}' must be >= {minimum}, got {v}")
        return v

    def number(self, key: str, default: Any = _MISSING) -> float:
        v = self._get(key, default)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{self.origin}: '{key}' must be a number, got {v!r}")
        return float(v)

    def boolean(self, key: str, default: Any = _MISSING) -> bool:
        v = self._get(key, default)
        if not isinstance(v, bool):
            raise ConfigError(f"{self.origin}: '{key}' must be true or false, got {v!r}")
        return v

    def string(self, key: str, default: Any = _MISSING) -> Any:
        v = self._get(key, default)
        if v is not None and not isinstance(v, str):
            raise ConfigError(f"{self.origin}: '{key}' must be a string, got {v!r}")
        return v

    def int_list(self, key: str, default: Any = _MISSING) -> List[int]:
        v = self._get(key, default)
        if isinstance(v, int) and not isinstance(v, bool):
            return [v]
        if not isinstance(v, (list, tuple)) or any(
                isinstance(x, bool) or not isinstance(x, int) for x in v):
            raise ConfigError(f"{self.origin}: '{key}' must be an integer or a list of integers")
        return list(v)


def read_config_json(model_dir: str) -> Tuple[Dict[str, Any], str]:
    """Return the parsed config.json of a model folder (or of the folder that
    holds a given .safetensors file) and its path."""
    folder = model_dir if os.path.isdir(model_dir) else os.path.dirname(model_dir)
    path = os.path.join(folder, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as fh:
            data = json.load(fh)
    except FileNotFoundError:
        raise ConfigError(f"cannot open config file: {path}") from None
    except json.JSONDecodeError as exc:
        raise ConfigError(f"{path}: not valid JSON ({exc})") from None
    return data, path
