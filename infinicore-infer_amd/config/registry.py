"""One registry from an architecture's name to its configuration class.

The reference picks the model with an if/elif chain over config["model_type"]
(scripts/jiuge.py:422,437,462,487) and raises ValueError("Unsupported model
architecture") (scripts/jiuge.py:502).  Here the chain is a table that any
module may extend with ``register_architecture``.
"""
import json
import os
from typing import Callable, Dict, Iterable, Type


class ConfigError(ValueError):
    """A config.json that cannot be turned into a typed configuration."""


_ARCHITECTURES: Dict[str, type] = {}


def register_architecture(names: Iterable[str], config_cls: type = None) -> Callable:
    """Register ``config_cls`` under each of ``names`` (values of ``model_type``
    or entries of ``architectures`` in config.json).  Usable as a decorator."""
    names = list(names)

    def _do(cls):
        for n in names:
            _ARCHITECTURES[n] = cls
        return cls

    if config_cls is not None:
        return _do(config_cls)
    return _do


def registered_architectures():
    return sorted(_ARCHITECTURES)


def resolve_architecture(config: dict) -> type:
    """Look the architecture up by ``model_type`` first, then by each entry of
    ``architectures``."""
    keys = []
    if "model_type" in config:
        keys.append(config["model_type"])
    keys.extend(config.get("architectures") or [])
    for k in keys:
        if k in _ARCHITECTURES:
            return _ARCHITECTURES[k]
    raise ConfigError(
        "Unsupported model architecture %r; registered: %s"
        % (keys, ", ".join(registered_architectures())))


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError("no config.json in %s" % model_dir)
    with open(path, "r", encoding="utf-8") as f:
        return json.load(f)


def config_from_dict(config: dict, **overrides):
    cls = resolve_architecture(config)
    return cls.from_dict(config, **overrides)


def config_from_dir(model_dir: str, **overrides):
    return config_from_dict(read_config_json(model_dir), **overrides)
