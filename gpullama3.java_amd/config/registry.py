"""One registry from the architecture's name (``architectures[0]`` of config.json, or its
``architecture`` where a folder names one as a plain string) to its typed configuration.

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
    if archs is None and isinstance(d.get("architecture"), str):
        archs = [d["architecture"]]
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
    if hasattr(cfg, "with_tensor_shapes"):
        # an architecture some of whose sizes only the weights give reads them from the files' headers
        cfg = cfg.with_tensor_shapes(_stored_shapes(folder))
    gen = os.path.join(folder, "generation_config.json")
    if os.path.isfile(gen) and not cfg.stop_ids:
        with open(gen) as f:
            cfg = cfg.with_stop_ids(_as_ids(json.load(f).get("eos_token_id")))
    return cfg


def _stored_shapes(folder):
    """Stored name -> shape of every tensor in the folder's safetensors files (headers only); {} without files."""
    from ..weights.loader import weight_files
    from ..weights.safetensors_io import SafetensorsFile
    out = {}
    try:
        paths = weight_files(folder)
    except FileNotFoundError:
        return out
    for p in paths:
        f = SafetensorsFile(p)
        try:
            for name in f.names():
                out[name] = tuple(f.shape(name))
        finally:
            f.close()
    return out


def _as_ids(v):
    if v is None:
        return ()
    if isinstance(v, int):
        return (v,)
    return tuple(int(i) for i in v)
