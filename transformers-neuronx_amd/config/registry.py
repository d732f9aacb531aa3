"""One registry from an architecture's name to its configuration and model.

The name is `config.json["architectures"][0]`; `model_type` is the fallback key,
as in the reference's `modeling_auto.py:5-47`, which keys on `model_type` and
asserts on an unknown one.
"""
import importlib
import json
import os
from dataclasses import dataclass
from typing import Any, Callable, Dict, List, Type, Union

from .model_config import ConfigError, ModelConfig


@dataclass
class Architecture:
    name: str                      # e.g. "OPTForCausalLM"
    model_type: str                # e.g. "opt"
    config_class: Type[ModelConfig]
    build_spec: Callable           # config -> parts.spec.ModelSpec
    # the user-facing class, or where it is found ("package.module:Class", imported when first asked for);
    # None: the architecture-free class serves
    model_class: Union[type, str, None] = None

    def user_class(self) -> type:
        if isinstance(self.model_class, str):
            module, _, name = self.model_class.partition(":")
            self.model_class = getattr(importlib.import_module(module), name)
        if self.model_class is None:
            from ..causal_lm import CausalLMForSampling
            return CausalLMForSampling
        return self.model_class


_ARCHITECTURES: Dict[str, Architecture] = {}

# Packages that register an architecture when they are imported. Another architecture is another package
# that calls `register_architecture`, and its name here (or a call of `add_architecture_package`, or just
# its import before a model folder is read). A program that is started apart (a command line) learns of
# packages from outside through the environment: TNX_ARCHITECTURE_PACKAGES holds module names, separated
# by commas, that are importable from where it runs.
ARCHITECTURE_PACKAGES: List[str] = ["transformers_neuronx_amd.opt"]
PACKAGES_VARIABLE = "TNX_ARCHITECTURE_PACKAGES"


def add_architecture_package(module: str) -> None:
    if module not in ARCHITECTURE_PACKAGES:
        ARCHITECTURE_PACKAGES.append(module)


def register_architecture(name: str, model_type: str, config_class, build_spec, model_class=None) -> Architecture:
    arch = Architecture(name, model_type, config_class, build_spec, model_class)
    _ARCHITECTURES[name] = arch
    return arch


def known_architectures():
    _load_builtin()
    return sorted(_ARCHITECTURES)


def _load_builtin():
    named = [m.strip() for m in os.environ.get(PACKAGES_VARIABLE, "").split(",") if m.strip()]
    for module in ARCHITECTURE_PACKAGES + named:
        try:
            importlib.import_module(module)
        except ImportError as e:
            if module in ARCHITECTURE_PACKAGES:
                raise
            raise ConfigError(f"{PACKAGES_VARIABLE} names '{module}', which cannot be imported: {e}") from e


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
