"""What every architecture's typed configuration shares, and how a ``config.json`` is read.

The base class carries only what every architecture has (its name and the raw
dictionary); each architecture adds a dataclass with the keys it reads, in its own
file under ``velox_amd/models`` (the reference has one hard-wired class,
``src/config.py:6-42``).
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


class ConfigError(ValueError):
    """A ``config.json`` that is missing a key, or holds one the engine refuses."""


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise ConfigError(f"no config.json in {model_dir!r}")
    with open(path, "r", encoding="utf-8") as handle:
        raw = json.load(handle)
    if not isinstance(raw, dict):
        raise ConfigError(f"{path}: expected a JSON object")
    return raw


def require(raw: Dict[str, Any], key: str, kind):
    if key not in raw or raw[key] is None:
        raise ConfigError(f"config.json is missing required key {key!r}")
    try:
        return kind(raw[key])
    except (TypeError, ValueError) as exc:
        raise ConfigError(f"config.json key {key!r}: cannot read {raw[key]!r} as {kind.__name__}") from exc


@dataclass
class ModelConfig:
    """What every architecture's configuration has in common."""

    architecture: str
    raw: Dict[str, Any] = field(repr=False, default_factory=dict)

    def to_json_dict(self) -> Dict[str, Any]:
        raise NotImplementedError


def read_generation_eos(model_dir: str) -> Optional[List[int]]:
    """EOS ids from ``generation_config.json`` when the folder has one (reference ``engine/engine.py:463-476``)."""
    path = os.path.join(model_dir, "generation_config.json")
    if not os.path.isfile(path):
        return None
    try:
        with open(path, "r", encoding="utf-8") as handle:
            eos = json.load(handle).get("eos_token_id")
    except (OSError, ValueError):
        return None
    if eos is None:
        return None
    return [int(eos)] if isinstance(eos, int) else [int(t) for t in eos]
