"""One registry from an architecture's name to its configuration class and model.

The reference keeps a map from the architecture string to what differs between
architectures and answers an unknown name with `unsupported model architecture %q`
(/root/reference/internal/llm/model.go:50-56, 77-81).  Here an entry holds the
class that parses config.json and the function that turns the parsed
configuration into a `ModelSpec` (the list of parts and their order).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable

from .base import ConfigError, read_config_json
from .specs import ModelSpec


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type                       # has from_dict(dict, where) and to_dict()
    model_spec: Callable[[object], ModelSpec]


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type, model_spec: Callable) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_class, model_spec)


def architecture_names() -> list[str]:
    return sorted(_ARCHITECTURES)


def lookup_architecture(name: str) -> Architecture:
    try:
        return _ARCHITECTURES[name]
    except KeyError:
        raise ConfigError(f'unsupported model architecture "{name}" '
                          f"(known: {', '.join(architecture_names()) or 'none'})") from None


def architecture_of(config_json: dict, where: str = "config.json") -> Architecture:
    archs = config_json.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError(f"{where}: key 'architectures' must be a list naming the model class")
    return lookup_architecture(archs[0])


def config_from_dict(config_json: dict, where: str = "config.json"):
    arch = architecture_of(config_json, where)
    return arch.config_class.from_dict(config_json, where)


def config_from_folder(model_dir: str):
    data = read_config_json(model_dir)
    return config_from_dict(data, where=f"{model_dir}/config.json")


def model_spec_of(config) -> ModelSpec:
    return lookup_architecture(config.architecture).model_spec(config)
