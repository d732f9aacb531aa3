"""Typed model configurations read from a checkpoint folder's config.json.

A configuration class lists the keys of its architecture's config.json, their
types and defaults; `from_dict` checks them and names the key at fault. Nothing
else in the package holds a model size. This module holds the base class only:
an architecture's configuration lives in the architecture's own package.
"""
import dataclasses
import json
import os
from dataclasses import dataclass
from typing import Any, ClassVar, Dict


class ConfigError(ValueError):
    """A config.json key is missing, of the wrong type, or out of range."""


REQUIRED = dataclasses.MISSING      # the default of a key that config.json must give


@dataclass(frozen=True)
class ModelConfig:
    """Base of the typed configurations: reading, checking, writing back."""

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, raw: Dict[str, Any]) -> "ModelConfig":
        values = {}
        for f in dataclasses.fields(cls):
            if f.name in raw and raw[f.name] is not None:
                values[f.name] = cls._coerce(f, raw[f.name])
            elif f.default is REQUIRED and f.default_factory is REQUIRED:
                raise ConfigError(f"config.json of {cls.architecture}: required key '{f.name}' is missing")
        cfg = cls(**values)
        cfg.validate()
        return cfg

    @classmethod
    def from_json(cls, path: str) -> "ModelConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as fp:
            return cls.from_dict(json.load(fp))

    @staticmethod
    def _coerce(f, value):
        want = f.type
        if want in ("int", int):
            if isinstance(value, bool) or not isinstance(value, int):
                raise ConfigError(f"key '{f.name}' must be an integer, got {value!r}")
            return value
        if want in ("float", float):
            if isinstance(value, bool) or not isinstance(value, (int, float)):
                raise ConfigError(f"key '{f.name}' must be a number, got {value!r}")
            return float(value)
        if want in ("bool", bool):
            if not isinstance(value, bool):
                raise ConfigError(f"key '{f.name}' must be true or false, got {value!r}")
            return value
        if want in ("str", str):
            if not isinstance(value, str):
                raise ConfigError(f"key '{f.name}' must be a string, got {value!r}")
            return value
        return value

    def validate(self) -> None:
        pass

    def to_dict(self) -> Dict[str, Any]:
        d = dataclasses.asdict(self)
        d["architectures"] = [self.architecture]
        return d

    def save(self, folder: str) -> None:
        os.makedirs(folder, exist_ok=True)
        with open(os.path.join(folder, "config.json"), "w") as fp:
            json.dump(self.to_dict(), fp, indent=2)
