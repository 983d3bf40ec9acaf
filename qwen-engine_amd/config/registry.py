"""One registry from the architecture name in config.json to its model.

An architecture is a function from the config.json dictionary to a typed
configuration object that has ``to_model_spec()`` and ``to_dict()``.
"""
from __future__ import annotations

import json
import os
from typing import Any, Callable, Dict

from .qwen3 import ARCHITECTURE as _QWEN3, ConfigError, Qwen3Config

_ARCHITECTURES: Dict[str, Callable[[Dict[str, Any]], Any]] = {}
_WANTS_SHAPES = set()


def register_architecture(name: str, from_dict: Callable[..., Any], tensor_shapes: bool = False) -> None:
    """``tensor_shapes``: some size of the design is given by a tensor's shape alone; ``from_dict`` then takes, as a
    second argument, the shapes of the model folder's tensors by name (none when there is no folder)."""
    _ARCHITECTURES[name] = from_dict
    if tensor_shapes:
        _WANTS_SHAPES.add(name)
    else:
        _WANTS_SHAPES.discard(name)


def unregister_architecture(name: str) -> None:
    _ARCHITECTURES.pop(name, None)
    _WANTS_SHAPES.discard(name)


def known_architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d: Dict[str, Any], shapes=None):
    archs = d.get("architectures") or ([d["architecture"]] if isinstance(d.get("architecture"), str) else None)
    if not archs:
        raise ConfigError("config.json has no 'architectures' (or 'architecture') entry; known: "
                          + ", ".join(known_architectures()))
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; known: "
                          + ", ".join(known_architectures()))
    if name in _WANTS_SHAPES:
        return _ARCHITECTURES[name](d, shapes() if callable(shapes) else (shapes or {}))
    return _ARCHITECTURES[name](d)


def folder_tensor_shapes(folder: str) -> Dict[str, tuple]:
    """name -> shape of every tensor in the folder's safetensors files, from their headers alone."""
    from safetensors import safe_open
    out: Dict[str, tuple] = {}
    for fn in sorted(os.listdir(folder)):
        if fn.endswith(".safetensors"):
            with safe_open(os.path.join(folder, fn), framework="pt", device="cpu") as f:
                for name in f.keys():
                    out[name] = tuple(f.get_slice(name).get_shape())
    return out


def config_from_folder(folder: str):
    path = os.path.join(folder, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {folder}")
    with open(path) as f:
        return config_from_dict(json.load(f), shapes=lambda: folder_tensor_shapes(folder))


register_architecture(_QWEN3, Qwen3Config.from_dict)


def _zarorax(d):
    from .zarorax import ZaroraxConfig
    return ZaroraxConfig.from_dict(d)


register_architecture("Zarorax", _zarorax)


def _nufavik(d):
    from .nufavik import NufavikConfig
    return NufavikConfig.from_dict(d)


register_architecture("Nufavik", _nufavik)


def _potatar(d, shapes=None):
    from .potatar import PotatarConfig
    return PotatarConfig.from_dict(d, shapes)


register_architecture("Potatar", _potatar, tensor_shapes=True)


def _safurax(d):
    from .safurax import SafuraxConfig
    return SafuraxConfig.from_dict(d)


register_architecture("Safurax", _safurax)
