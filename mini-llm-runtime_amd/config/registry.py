"""One registry from an architecture's name (config.json `architectures[0]`) to its
configuration class.  The configuration class knows the architecture's config.json keys, its
tensor names and how to describe itself as a `ModelSpec`."""
from __future__ import annotations

import json
import os

_ARCHITECTURES = {}


class ConfigError(ValueError):
    pass


def register_architecture(name):
    def add(cls):
        _ARCHITECTURES[name] = cls
        cls.architecture = name
        return cls
    return add


def known_architectures():
    return sorted(_ARCHITECTURES)


def config_class(name):
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture {name!r}; known: {', '.join(known_architectures()) or 'none'}")
    return _ARCHITECTURES[name]


def config_from_dict(data):
    archs = data.get("architectures")
    if not isinstance(archs, list) or len(archs) != 1 or not isinstance(archs[0], str):
        raise ConfigError("config.json needs `architectures` with exactly one name")
    return config_class(archs[0]).from_dict(data)


def load_config(folder):
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder}")
    with open(path) as f:
        try:
            data = json.load(f)
        except json.JSONDecodeError as err:
            raise ConfigError(f"{path}: not valid JSON ({err})") from None
    if not isinstance(data, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return config_from_dict(data)
