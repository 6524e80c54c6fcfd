"""One registry from an architecture's name to its configuration class and
its model builder.

The reference has no registry: it treats every model_type that does not start
with "gemma3" as Llama and never consults ``architectures``
(models/config.go:152-153).  Here the name in ``architectures[0]`` selects the
entry; an unknown name is an error that lists the registered ones.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict

from .base import ConfigError, ModelConfig, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type
    build: Callable  # (config) -> kllm_amd.parts.spec.ModelSpec
    model_types: tuple = ()


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name, config_class, build, model_types=()):
    """Make ``name`` (as written in config.json's ``architectures``) loadable.
    ``build(config)`` returns the model's ModelSpec: its parts, layer list and
    running order."""
    _ARCHITECTURES[name] = Architecture(name, config_class, build, tuple(model_types))
    return _ARCHITECTURES[name]


def unregister_architecture(name):
    _ARCHITECTURES.pop(name, None)


def registered_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(raw: dict, where: str = "config.json") -> Architecture:
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs:
        name = archs[0]
        if name in _ARCHITECTURES:
            return _ARCHITECTURES[name]
        raise ConfigError(
            f"{where}: architecture {name!r} is not registered "
            f"(registered: {', '.join(registered_architectures()) or 'none'})")
    mtype = raw.get("model_type")
    for arch in _ARCHITECTURES.values():
        if mtype is not None and mtype in arch.model_types:
            return arch
    raise ConfigError(
        f"{where}: no 'architectures' entry and model_type {mtype!r} is unknown "
        f"(registered: {', '.join(registered_architectures()) or 'none'})")


def config_from_dict(raw: dict, where: str = "config.json") -> ModelConfig:
    arch = resolve_architecture(raw, where)
    return arch.config_class.from_dict(raw, where)


def load_config(model_dir: str) -> ModelConfig:
    """Read ``model_dir/config.json`` into the typed configuration of the
    architecture it names."""
    raw = read_config_json(model_dir)
    return config_from_dict(raw, where=f"{model_dir}/config.json")
