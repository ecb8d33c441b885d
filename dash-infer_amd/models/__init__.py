"""Model registry: config.json -> the class that serves it.

    @register("Name")            a class with  from_config(config, tensors, state, dtype)  and the forward interface of
                                 the sequence engine (models/modanex.py), or a config translator for the decode runner
    resolve(config)              by config["architecture"] / ["architectures"][0] / ["model_type"]
    load(path, ...)              config.json + model.safetensors of a folder -> (model class, config, tensors)
"""
import json
import os

_REGISTRY = {}


def register(*names):
    def deco(cls):
        for n in names:
            _REGISTRY[n] = cls
        return cls
    return deco


def architecture_of(config):
    if "architecture" in config:
        return config["architecture"]
    if config.get("architectures"):
        return config["architectures"][0]
    if "model_type" in config:
        return config["model_type"]
    raise KeyError("config.json names no architecture")


def resolve(config):
    _load_builtin()
    name = architecture_of(config)
    if name not in _REGISTRY:
        raise KeyError(f"no model class registered for architecture {name!r} (known: {sorted(_REGISTRY)})")
    return _REGISTRY[name]


def known():
    _load_builtin()
    return sorted(_REGISTRY)


def read_config(path):
    with open(os.path.join(path, "config.json")) as f:
        return json.load(f)


def _load_builtin():
    from . import filipel, modanex, qwen2, tobilorn, vogusun  # noqa: F401  (registration on import)
