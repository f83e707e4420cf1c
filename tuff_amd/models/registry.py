"""One table from an architecture's name (config.json `architectures[0]`) to its configuration
class and the function that builds its model.  The reference keeps the same table as an enum
plus a switch over engine vtables (include/tuff_vtable.h:13-57, src/tuff_vtable.c:159-171).
"""
from __future__ import annotations

import dataclasses
from typing import Callable, Type

from ..config.base import ConfigError, ModelConfig, architecture_name, read_config_json


@dataclasses.dataclass(frozen=True)
class Architecture:
    name: str
    config_cls: Type[ModelConfig]
    build: Callable[[ModelConfig], "object"]      # -> DecoderModel


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(name: str, config_cls: Type[ModelConfig], build: Callable) -> None:
    if name in _ARCHITECTURES:
        raise ValueError(f"architecture '{name}' is already registered")
    _ARCHITECTURES[name] = Architecture(name, config_cls, build)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)


def get_architecture(name: str) -> Architecture:
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture '{name}'; registered: {sorted(_ARCHITECTURES)}")
    return _ARCHITECTURES[name]


def architectures() -> list[str]:
    return sorted(_ARCHITECTURES)


def config_from_dict(raw: dict) -> ModelConfig:
    return get_architecture(architecture_name(raw)).config_cls.from_dict(raw)


def load_config(model_dir: str) -> ModelConfig:
    return config_from_dict(read_config_json(model_dir))


def build_model(cfg: ModelConfig):
    return get_architecture(cfg.architecture).build(cfg)


def _register_builtin() -> None:
    from ..config.lfm2 import Lfm2Config
    from .lfm2 import build_lfm2
    register_architecture(Lfm2Config.architecture, Lfm2Config, build_lfm2)


_register_builtin()
