"""One registry from the architecture's name (config.json "model_type") to its configuration
class.  The reference's counterpart accepts exactly "llama"
(src/libllm/model_for_generation.cc:33-52); adding an architecture is one ``register`` call."""
import json
import os
from typing import Any, Dict

from ..errors import ConfigError

_ARCHITECTURES: Dict[str, Any] = {}


def register_architecture(model_type: str, config_class) -> None:
    """``config_class`` must offer ``from_dict(dict)`` and instances with ``to_spec()`` (the
    model as data) and ``to_dict()`` (config.json again)."""
    _ARCHITECTURES[model_type] = config_class


def architectures():
    return sorted(_ARCHITECTURES)


def config_from_dict(d: Dict[str, Any]):
    if not isinstance(d, dict):
        raise ConfigError("config.json must hold an object")
    model_type = d.get("model_type")
    if not isinstance(model_type, str):
        raise ConfigError("config.json: required key 'model_type' is missing")
    if model_type not in _ARCHITECTURES:
        raise ConfigError("unexpected model type: %s (registered: %s)"
                          % (model_type, ", ".join(architectures())))
    return _ARCHITECTURES[model_type].from_dict(d)


def config_from_dir(model_dir: str):
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError("no config.json in %s" % model_dir)
    try:
        with open(path, "r", encoding="utf-8") as f:
            d = json.load(f)
    except json.JSONDecodeError as e:
        raise ConfigError("%s is not valid JSON: %s" % (path, e))
    return config_from_dict(d)
