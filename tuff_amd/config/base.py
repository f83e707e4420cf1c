"""Typed model configurations read from an architecture's own config.json keys.

A configuration class lists its keys as dataclass fields (name = config.json key),
converts and checks them in `validate`, and writes them back with `to_dict`, so that
a folder written from a configuration reads back to the same configuration.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, ClassVar


class ConfigError(ValueError):
    """A config.json that cannot be used: missing key, wrong type, inconsistent sizes."""


_REQUIRED = dataclasses.MISSING


@dataclasses.dataclass
class ModelConfig:
    """Base of every architecture's configuration.

    Subclasses add fields; a field without default is a required key.  `aliases`
    maps alternative config.json spellings to field names.
    """

    architecture: ClassVar[str] = ""
    aliases: ClassVar[dict[str, str]] = {}
    # keys that may appear in config.json and carry nothing the engine needs
    ignored: ClassVar[frozenset[str]] = frozenset({
        "architectures", "model_type", "torch_dtype", "dtype", "transformers_version",
        "use_cache", "initializer_range", "_name_or_path", "use_pos_enc", "auto_map",
    })

    @classmethod
    def from_dict(cls, raw: dict[str, Any]) -> "ModelConfig":
        fields = {f.name: f for f in dataclasses.fields(cls)}
        values: dict[str, Any] = {}
        unknown = []
        for key, val in raw.items():
            name = cls.aliases.get(key, key)
            if name in fields:
                if name in values and key != name:
                    continue            # the canonical spelling wins over an alias
                values[name] = val
            elif key not in cls.ignored:
                unknown.append(key)
        missing = [n for n, f in fields.items()
                   if n not in values and f.default is _REQUIRED and f.default_factory is _REQUIRED]
        if missing:
            raise ConfigError(f"{cls.architecture or cls.__name__}: config.json lacks required "
                              f"key(s): {', '.join(sorted(missing))}")
        cfg = cls(**values)
        cfg.unknown_keys = sorted(unknown)
        cfg.validate()
        return cfg

    def validate(self) -> None:                      # pragma: no cover - overridden
        pass

    def to_dict(self) -> dict[str, Any]:
        out = {"architectures": [self.architecture]}
        out.update(dataclasses.asdict(self))
        return out

    # -- helpers for subclasses ---------------------------------------------------
    def _int(self, name: str, minimum: int = 1) -> None:
        v = getattr(self, name)
        if isinstance(v, bool) or not isinstance(v, int):
            if isinstance(v, float) and v == int(v):
                v = int(v)
            else:
                raise ConfigError(f"{name} must be an integer, got {v!r}")
        if v < minimum:
            raise ConfigError(f"{name} must be >= {minimum}, got {v}")
        setattr(self, name, v)

    def _float(self, name: str, positive: bool = True) -> None:
        v = getattr(self, name)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{name} must be a number, got {v!r}")
        v = float(v)
        if positive and not v > 0.0:
            raise ConfigError(f"{name} must be > 0, got {v}")
        setattr(self, name, v)

    def _bool(self, name: str) -> None:
        v = getattr(self, name)
        if not isinstance(v, bool):
            raise ConfigError(f"{name} must be true or false, got {v!r}")


def read_config_json(model_dir: str) -> dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {model_dir}")
    with open(path) as f:
        try:
            raw = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return raw


def architecture_name(raw: dict[str, Any]) -> str:
    archs = raw.get("architectures")
    if isinstance(archs, list) and archs and isinstance(archs[0], str):
        return archs[0]
    raise ConfigError("config.json has no 'architectures' list naming the model class")
