"""One registry from an architecture's name (config.json ``architectures[0]``)
to its configuration class and its model builder.

The reference has no such table: its runner holds a ``Qwen3`` member
(src/engine/model_runner.hpp:21, src/engine/model_runner.cpp:29)."""
from __future__ import annotations

import json
import os
from typing import Callable, Dict, NamedTuple, Type

from .model_config import ConfigError, ModelConfig


class Architecture(NamedTuple):
    name: str
    config_cls: Type[ModelConfig]
    #: build(config) -> spyinfer_amd.models.base.DecoderModel (weights not yet bound)
    build: Callable


_REGISTRY: Dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig], build: Callable) -> None:
    _REGISTRY[name] = Architecture(name, config_cls, build)


def unregister_architecture(name: str) -> None:
    _REGISTRY.pop(name, None)


def registered_architectures():
    _load_builtin()
    return sorted(_REGISTRY)


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    if name not in _REGISTRY:
        raise ConfigError("architecture %r is not registered; known: %s" % (name, ", ".join(sorted(_REGISTRY)) or "(none)"))
    return _REGISTRY[name]


def architecture_of(raw: dict) -> Architecture:
    archs = raw.get("architectures")
    if not isinstance(archs, list) or not archs or not isinstance(archs[0], str):
        raise ConfigError("config.json lacks 'architectures': [name]; known: %s" % ", ".join(registered_architectures()))
    return get_architecture(archs[0])


def load_model_config(folder: str):
    """Read ``folder/config.json`` -> (Architecture, typed configuration)."""
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError("no config.json in %s" % folder)
    with open(path) as f:
        raw = json.load(f)
    arch = architecture_of(raw)
    return arch, arch.config_cls.from_dict(raw)


def _load_builtin() -> None:
    # Importing the models package registers the architectures that ship with the engine.
    from .. import models  # noqa: F401
