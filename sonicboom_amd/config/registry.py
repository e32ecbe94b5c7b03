"""The one registry from an architecture's name to its model.

An architecture registers the name config.json carries in ``architectures[0]``
together with its typed configuration class and a function that turns a
configuration into a :class:`~sonicboom_amd.parts.spec.ModelSpec`.  Everything
else in the framework (loader, engine, tools) goes through this table; the
reference does the same with a switch over ``general.architecture``
(/root/reference/core/src/model/loader.cpp:847-865, :1128-1141).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Mapping

from .base import ConfigError, merge_generation_config, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    config_class: type          # has from_dict(dict) and to_dict()
    build_spec: Callable        # config -> ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, config_class: type, build_spec: Callable) -> None:
    _ARCHITECTURES[name] = Architecture(name, config_class, build_spec)


def registered_architectures():
    _load_builtin()
    return sorted(_ARCHITECTURES)


def _load_builtin() -> None:
    from .. import architectures  # noqa: F401  (registers on import)


def architecture_of(config: Mapping) -> Architecture:
    """The registered architecture a config.json dict names."""
    _load_builtin()
    names = config.get("architectures")
    if not isinstance(names, (list, tuple)) or not names or not isinstance(names[0], str):
        raise ConfigError("missing/invalid config key: architectures (want a list with the model class name)")
    arch = _ARCHITECTURES.get(names[0])
    if arch is None:
        raise ConfigError(f"unknown architecture: {names[0]} (registered: {', '.join(sorted(_ARCHITECTURES))})")
    return arch


def load_config(folder: str):
    """(architecture, typed configuration) of a model folder."""
    d = merge_generation_config(folder, read_config_json(folder))
    arch = architecture_of(d)
    return arch, arch.config_class.from_dict(d)
