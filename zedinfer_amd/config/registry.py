"""One registry from an architecture's name to its model.

The reference dispatches on ``model_type`` with an if/else chain
(reference: src/frontend/models/base.cpp:419-463, :807-926) and throws
"Unsupported model type" otherwise.  Here an architecture registers a config
class and a function that turns that config into a ``ModelForwardConfig``;
``architectures[0]`` of config.json is the key and ``model_type`` an alias.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict, Mapping, Tuple, Type

from .forward_config import ModelForwardConfig
from .model_config import ConfigError, ModelConfig, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Type[ModelConfig]
    forward_config: Callable[[ModelConfig], ModelForwardConfig]
    aliases: Tuple[str, ...] = ()


_ARCHITECTURES: Dict[str, Architecture] = {}
_ALIASES: Dict[str, str] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig],
                          forward_config: Callable[[Any], ModelForwardConfig],
                          aliases: Tuple[str, ...] = ()) -> Architecture:
    arch = Architecture(name, config_cls, forward_config, tuple(aliases))
    _ARCHITECTURES[name] = arch
    for a in aliases:
        _ALIASES[a] = name
    return arch


def registered_architectures() -> Tuple[str, ...]:
    return tuple(sorted(_ARCHITECTURES))


def find_architecture(config_dict: Mapping[str, Any]) -> Architecture:
    archs = config_dict.get("architectures") or []
    for a in archs:
        if a in _ARCHITECTURES:
            return _ARCHITECTURES[a]
    mt = config_dict.get("model_type")
    if mt in _ALIASES:
        return _ARCHITECTURES[_ALIASES[mt]]
    raise ConfigError(
        f"unsupported architecture: architectures={list(archs)!r}, model_type={mt!r}; "
        f"registered: {', '.join(registered_architectures()) or '(none)'}")


def load_config(path: str) -> Tuple[Architecture, ModelConfig]:
    """Read a model folder's config.json and return its architecture and typed config."""
    d = read_config_json(path)
    arch = find_architecture(d)
    return arch, arch.config_cls.from_dict(d)
