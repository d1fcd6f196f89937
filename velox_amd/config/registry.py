"""One registry from the model class named in ``config.json`` to how it is built.

The reference builds its single class directly (``engine/engine.py:130``); here an
architecture registers a configuration reader and a function that turns the
configuration into a :class:`~velox_amd.parts.model.ModelSpec`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict

from .model_config import ConfigError, ModelConfig, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[Dict[str, Any]], ModelConfig]
    make_spec: Callable[..., Any]  # (config, max_position) -> ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}
_ARCHITECTURE_OF_MODEL_TYPE: Dict[str, str] = {}


def register_architecture(name: str, read_config, make_spec, model_types=()) -> None:
    """``name`` is what ``config.json`` holds in ``architectures[0]``; ``model_types`` are values of its ``model_type``
    key that stand for this class when ``architectures`` is left out."""
    _ARCHITECTURES[name] = Architecture(name, read_config, make_spec)
    for model_type in model_types:
        _ARCHITECTURE_OF_MODEL_TYPE[model_type] = name


def architecture_name(raw: Dict[str, Any]) -> str:
    names = raw.get("architectures")
    if names and isinstance(names, (list, tuple)) and isinstance(names[0], str):
        return names[0]
    _load_builtin()
    model_type = raw.get("model_type")
    if isinstance(model_type, str) and model_type in _ARCHITECTURE_OF_MODEL_TYPE:
        return _ARCHITECTURE_OF_MODEL_TYPE[model_type]
    raise ConfigError('config.json must name its model class in "architectures" (or a known "model_type")')


def known_architectures():
    return sorted(_ARCHITECTURES)


def get_architecture(name: str) -> Architecture:
    _load_builtin()
    if name not in _ARCHITECTURES:
        raise ConfigError(f"unknown architecture {name!r}; registered: {known_architectures()}")
    return _ARCHITECTURES[name]


def config_from_dict(raw: Dict[str, Any]) -> ModelConfig:
    return get_architecture(architecture_name(raw)).read_config(raw)


def load_config(model_dir: str) -> ModelConfig:
    return config_from_dict(read_config_json(model_dir))


def _load_builtin() -> None:
    from .. import models  # noqa: F401  (registers the built-in architectures)
