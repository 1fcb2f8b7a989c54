"""One registry from an architecture's name to its typed config.

`config.json["architectures"][0]` is the key, as in model folders of this kind. An
architecture is a class with `from_dict(config_json) -> config` and
`config.model_spec() -> ModelSpec`; everything else is built from parts. The
reference hard-wires its one class (worker/src/inference/torch_engine.py:142).
"""

from __future__ import annotations

from typing import Any, Dict, Mapping

from .model_config import ConfigError, ModelSpec, Qwen2Config, read_config_json

_ARCHITECTURES: Dict[str, Any] = {}


def register_architecture(name: str, config_class) -> None:
    """`config_class.from_dict(dict)` must return an object with `model_spec()`."""
    if not hasattr(config_class, "from_dict"):
        raise TypeError("an architecture config needs a from_dict(config_json) classmethod")
    _ARCHITECTURES[name] = config_class


def known_architectures() -> list:
    return sorted(_ARCHITECTURES)


def architecture_of(config_json: Mapping[str, Any]) -> str:
    names = config_json.get("architectures")
    if not names or not isinstance(names, (list, tuple)):
        raise ConfigError("config.json lacks 'architectures'; known: " + ", ".join(known_architectures()))
    name = str(names[0])
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; known: " + ", ".join(known_architectures()))
    return name


def config_from_dict(config_json: Mapping[str, Any]):
    return _ARCHITECTURES[architecture_of(config_json)].from_dict(config_json)


def load_model_config(model_dir):
    """The typed config of the model folder `model_dir`."""
    return config_from_dict(read_config_json(model_dir))


def model_spec_from_dir(model_dir) -> ModelSpec:
    return load_model_config(model_dir).model_spec()


register_architecture(Qwen2Config.architecture, Qwen2Config)
