"""One registry from the architecture's name (``architectures[0]`` of config.json)
to its typed configuration.

The reference maps an enum constant to a loader and throws for an unknown type
(J/model/ModelType.java:24-75); here the key is the name the model folder itself
carries, and an unknown name lists the registered ones.
"""
from __future__ import annotations

import json
import os

_ARCHITECTURES = {}


class ConfigError(ValueError):
    """A config.json that the engine cannot run; the message names the key."""


def register_architecture(name, config_cls):
    """``config_cls`` needs ``from_dict(dict)``, ``to_dict()`` and ``model_spec()``."""
    _ARCHITECTURES[name] = config_cls
    return config_cls


def registered_architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d):
    archs = d.get("architectures")
    if not isinstance(archs, (list, tuple)) or not archs:
        raise ConfigError("config.json: 'architectures' is missing or empty; "
                          f"registered: {registered_architectures()}")
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(f"config.json: unknown architecture {name!r}; "
                          f"registered: {registered_architectures()}")
    return _ARCHITECTURES[name].from_dict(d)


def load_config(folder):
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"no config.json in {folder}")
    with open(path) as f:
        d = json.load(f)
    cfg = config_from_dict(d)
    gen = os.path.join(folder, "generation_config.json")
    if os.path.isfile(gen) and not cfg.stop_ids:
        with open(gen) as f:
            cfg = cfg.with_stop_ids(_as_ids(json.load(f).get("eos_token_id")))
    return cfg


def _as_ids(v):
    if v is None:
        return ()
    if isinstance(v, int):
        return (v,)
    return tuple(int(i) for i in v)
