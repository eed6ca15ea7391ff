"""The one registry from an architecture's name to its model.

``architectures[0]`` of config.json selects an entry; an entry holds the typed
configuration class and the builder that turns a configuration into a
``ModelSpec``.  An unknown name is an error that lists the known ones, as the
reference refuses a GGUF architecture that is not on its allowlist
(src/model.c:751-763, :1395-1418).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping

from .base import ConfigError, architecture_name, read_config_json
from .spec import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    parse_config: Callable[[Mapping[str, Any]], Any]
    build_spec: Callable[[Any], ModelSpec]


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, parse_config: Callable[[Mapping[str, Any]], Any],
                          build_spec: Callable[[Any], ModelSpec], replace: bool = False) -> None:
    if name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {name!r} is already registered")
    _ARCHITECTURES[name] = Architecture(name, parse_config, build_spec)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def known_architectures() -> list:
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(
            f"architecture {name!r} is not supported; known: {', '.join(known_architectures()) or '(none)'}"
        ) from None


def load_config(model_dir: str):
    """Read ``model_dir/config.json`` -> (architecture entry, typed config)."""
    raw = read_config_json(model_dir)
    arch = get_architecture(architecture_name(raw))
    return arch, arch.parse_config(raw)


def config_from_dict(raw: Mapping[str, Any]):
    arch = get_architecture(architecture_name(raw))
    return arch, arch.parse_config(raw)
