"""Configurations and the one registry from an architecture's name to its model.

An entry couples the name that config.json carries in ``architectures[0]`` with
a typed configuration class.  The class parses config.json (``from_dict``),
writes it back (``to_dict``) and describes the model as parts (``to_spec``);
the generic decoder is assembled from that description, so registering a
configuration class registers the model.
"""

from __future__ import annotations

import json
import os
from typing import Any, Callable, Dict, Mapping

from .spec import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec  # noqa: F401
from .lfm2 import Lfm2Config, feed_forward_width  # noqa: F401

_ARCHITECTURES: Dict[str, Any] = {}


def register_architecture(name: str, config_class: Any) -> None:
    """``config_class`` needs ``from_dict(mapping)`` and ``to_spec()``."""
    for attr in ("from_dict", "to_spec"):
        if not hasattr(config_class, attr):
            raise TypeError(f"{config_class!r} lacks {attr}()")
    _ARCHITECTURES[name] = config_class


def known_architectures() -> list:
    return sorted(_ARCHITECTURES)


def config_from_dict(data: Mapping[str, Any]):
    archs = data.get("architectures")
    if not archs or not isinstance(archs, (list, tuple)) or not isinstance(archs[0], str):
        raise ConfigError(
            "config.json has no architectures entry; known architectures: "
            + ", ".join(known_architectures()))
    name = archs[0]
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unsupported architecture {name!r}; known architectures: "
            + ", ".join(known_architectures()))
    return _ARCHITECTURES[name].from_dict(data)


def load_config(model_dir: str):
    """Read ``model_dir/config.json`` (or the JSON file ``model_dir`` itself) and parse
    it with the registered class."""
    path = model_dir if os.path.isfile(model_dir) else os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"{path} does not exist")
    with open(path, "r", encoding="utf-8") as f:
        try:
            data = json.load(f)
        except json.JSONDecodeError as e:
            raise ConfigError(f"{path} is not valid JSON: {e}") from e
    if not isinstance(data, dict):
        raise ConfigError(f"{path} does not hold a JSON object")
    return config_from_dict(data)


register_architecture("Lfm2ForCausalLM", Lfm2Config)
