"""One registry from an architecture's name to its configuration and model.

The name is `config.json["architectures"][0]`; `model_type` is the fallback key,
as in the reference's `modeling_auto.py:5-47`, which keys on `model_type` and
asserts on an unknown one.
"""
import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, Optional, Type

from .model_config import ConfigError, ModelConfig


@dataclass
class Architecture:
    name: str                      # e.g. "OPTForCausalLM"
    model_type: str                # e.g. "opt"
    config_class: Type[ModelConfig]
    build_spec: Callable           # config -> parts.spec.ModelSpec
    model_class: Optional[type] = None   # user-facing class (set when its module is imported)


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, model_type: str, config_class, build_spec, model_class=None) -> Architecture:
    arch = Architecture(name, model_type, config_class, build_spec, model_class)
    _ARCHITECTURES[name] = arch
    return arch


def known_architectures():
    _load_builtin()
    return sorted(_ARCHITECTURES)


def _load_builtin():
    # The built-in architectures register themselves on import.
    from .. import opt  # noqa: F401


def resolve(raw: Dict[str, Any]) -> Architecture:
    """The architecture a config.json names."""
    _load_builtin()
    names = raw.get("architectures") or []
    for n in names:
        if n in _ARCHITECTURES:
            return _ARCHITECTURES[n]
    mt = raw.get("model_type")
    for arch in _ARCHITECTURES.values():
        if mt is not None and arch.model_type == mt:
            return arch
    raise ConfigError(
        f"config.json names architectures {names!r} and model_type {mt!r}; "
        f"known architectures: {sorted(_ARCHITECTURES)}")


def read_config(folder_or_file: str):
    """(architecture, typed config) of a model folder."""
    path = folder_or_file
    if os.path.isdir(path):
        path = os.path.join(path, "config.json")
    if not os.path.exists(path):
        raise FileNotFoundError(f"no config.json at {path}")
    with open(path) as fp:
        raw = json.load(fp)
    arch = resolve(raw)
    return arch, arch.config_class.from_dict(raw)
