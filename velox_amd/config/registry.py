"""One registry from the model class named in ``config.json`` to how it is built.

The reference builds its single class directly (``engine/engine.py:130``); here an
architecture registers a configuration reader and a function that turns the
configuration into a :class:`~velox_amd.parts.model.ModelSpec`.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Dict

from .model_config import ConfigError, ModelConfig, architecture_name, read_config_json


@dataclass(frozen=True)
class Architecture:
    name: str
    read_config: Callable[[Dict[str, Any]], ModelConfig]
    make_spec: Callable[..., Any]  # (config, max_position) -> ModelSpec


_ARCHITECTURES: Dict[str, Architecture] = {}


def register_architecture(name: str, read_config, make_spec) -> None:
    _ARCHITECTURES[name] = Architecture(name, read_config, make_spec)


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
