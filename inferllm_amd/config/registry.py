"""One registry from an architecture's name (config.json `architectures[0]`) to
its configuration class.  The configuration class reads the architecture's own
config.json keys and translates itself into a `ModelSpec`.

The reference keeps the same idea as an if/else chain over a model-type string
(src/graph/graph_imp.cpp:6-21, unknown name: assert "unsupported model").
"""
from __future__ import annotations

import json
import os
from typing import Callable, Dict


class ConfigError(ValueError):
    """A config.json that cannot be served: missing key, bad value, unknown option."""


_ARCHITECTURES: Dict[str, type] = {}


def register_architecture(name: str) -> Callable[[type], type]:
    """Class decorator: `@register_architecture("LlamaForCausalLM")`."""
    def deco(cls: type) -> type:
        if name in _ARCHITECTURES and _ARCHITECTURES[name] is not cls:
            raise ConfigError(f"architecture {name!r} is already registered")
        _ARCHITECTURES[name] = cls
        cls.architecture = name
        return cls
    return deco


def registered_architectures():
    return sorted(_ARCHITECTURES)


def config_class(name: str) -> type:
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unsupported architecture {name!r}; registered: {registered_architectures()}")
    return _ARCHITECTURES[name]


def config_from_dict(d: dict):
    """Typed configuration from the dict of a config.json."""
    archs = d.get("architectures")
    if not isinstance(archs, (list, tuple)) or len(archs) == 0 or not isinstance(archs[0], str):
        raise ConfigError("config.json needs `architectures`: a list with the model class name; "
                          f"registered: {registered_architectures()}")
    return config_class(archs[0]).from_dict(d)


def load_config(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {model_dir!r}")
    with open(path, "r", encoding="utf-8") as f:
        try:
            d = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path}: not valid JSON ({e})") from None
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level must be an object")
    return config_from_dict(d)
