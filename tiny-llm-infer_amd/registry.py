"""The one registry from an architecture's name (``architectures[0]`` of its
config.json) to what builds it: a typed configuration reader and a function
that turns that configuration into an architecture-neutral ``ModelSpec``.

The reference has no registry; it constructs its one model class directly
(utils/include/status.h:41-45 holds only an enum with a single entry)."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict

from .config.base import ConfigError, ModelSpec, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[Dict[str, Any], str], Any]   # (json dict, origin) -> typed config
    make_spec: Callable[[Any], ModelSpec]               # typed config -> ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, read_config, make_spec, replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, read_config, make_spec)


def architecture_names():
    return sorted(_ARCHITECTURES)


def lookup_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f"architecture '{name}' is not registered; known: "
                          f"{', '.join(architecture_names()) or 'none'}") from None


def architecture_of(config_json: Dict[str, Any], origin: str = "config.json") -> Architecture:
    archs = config_json.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError(f"{origin}: 'architectures' must be a non-empty list of names")
    return lookup_architecture(archs[0])


def load_config(model_dir: str):
    """Read config.json of ``model_dir``; return (architecture, typed config)."""
    data, path = read_config_json(model_dir)
    arch = architecture_of(data, path)
    return arch, arch.read_config(data, path)
