"""Typed model configuration, read straight from a model folder's ``config.json``.

The base class carries only what every architecture has (its name and the raw
dictionary); each architecture adds a dataclass with the keys it reads.  The
Qwen2 keys and their defaults follow the reference's ``ModelConfig.from_hf``
(reference ``src/config.py:29-42``); unlike the reference, keys that change the
arithmetic and that the engine does not implement are refused instead of
ignored (the reference never reads ``use_sliding_window`` or ``hidden_act`` and
silently ignores non-linear ``rope_scaling``, ``src/rope.py:11-18``).
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


# model classes by "model_type", for a config.json that leaves "architectures" out
_CLASS_OF_MODEL_TYPE = {"qwen2": "Qwen2ForCausalLM"}


def architecture_name(raw: Dict[str, Any]) -> str:
    names = raw.get("architectures")
    if names and isinstance(names, (list, tuple)) and isinstance(names[0], str):
        return names[0]
    model_type = raw.get("model_type")
    if isinstance(model_type, str) and model_type in _CLASS_OF_MODEL_TYPE:
        return _CLASS_OF_MODEL_TYPE[model_type]
    raise ConfigError('config.json must name its model class in "architectures" (or a known "model_type")')


def _require(raw: Dict[str, Any], key: str, kind):
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


@dataclass
class Qwen2Config(ModelConfig):
    """Qwen2 / Qwen2.5 dense decoder (reference ``src/config.py:6-42``)."""

    hidden_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    intermediate_size: int = 0
    rms_norm_eps: float = 0.0
    vocab_size: int = 0
    max_position_embeddings: int = 0
    rope_theta: float = 0.0
    rope_scaling_factor: float = 1.0
    tie_word_embeddings: bool = False
    eos_token_ids: List[int] = field(default_factory=list)

    @staticmethod
    def from_dict(raw: Dict[str, Any]) -> "Qwen2Config":
        hidden = _require(raw, "hidden_size", int)
        heads = _require(raw, "num_attention_heads", int)
        # reference src/config.py:34: kv heads default to the query heads
        kv_heads = int(raw.get("num_key_value_heads") or heads)
        if heads <= 0 or kv_heads <= 0 or heads % kv_heads != 0:
            raise ConfigError(
                f"num_attention_heads={heads} must be a positive multiple of num_key_value_heads={kv_heads}"
            )
        # reference src/self_attention.py:28 computes hidden // heads; a stored head_dim wins
        if raw.get("head_dim") is not None:
            head_dim = int(raw["head_dim"])
        else:
            if hidden % heads != 0:
                raise ConfigError(f"hidden_size={hidden} is not divisible by num_attention_heads={heads}")
            head_dim = hidden // heads
        if head_dim <= 0 or head_dim % 2 != 0:
            raise ConfigError(f"head_dim={head_dim} must be positive and even (rotary halves)")

        # reference src/config.py:36,38,39
        eps = float(raw.get("rms_norm_eps", raw.get("layer_norm_eps", 1e-6)))
        max_pos = int(raw.get("max_position_embeddings", raw.get("seq_length", 4096)))
        theta = float(raw.get("rope_theta", 10000.0))

        factor = 1.0
        scaling = raw.get("rope_scaling")
        if scaling:
            # reference src/rope.py:11-18: only linear scaling divides the positions
            kind = scaling.get("type") or scaling.get("rope_type")
            if kind in (None, "default"):
                factor = 1.0
            elif kind == "linear":
                factor = float(scaling.get("factor", 1.0))
                if factor <= 0:
                    raise ConfigError(f"rope_scaling.factor={factor} must be positive")
            else:
                raise ConfigError(f"rope_scaling type {kind!r} is not implemented (only 'linear')")

        if raw.get("use_sliding_window"):
            raise ConfigError("use_sliding_window=true is not implemented for Qwen2 (every layer attends to all keys)")
        act = raw.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"hidden_act={act!r} is not implemented for Qwen2 (only 'silu')")

        eos = raw.get("eos_token_id")
        if eos is None:
            eos_ids: List[int] = []
        elif isinstance(eos, int):
            eos_ids = [eos]
        else:
            eos_ids = [int(t) for t in eos]

        cfg = Qwen2Config(
            architecture=architecture_name(raw),
            raw=dict(raw),
            hidden_size=hidden,
            num_hidden_layers=_require(raw, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=_require(raw, "intermediate_size", int),
            rms_norm_eps=eps,
            vocab_size=_require(raw, "vocab_size", int),
            max_position_embeddings=max_pos,
            rope_theta=theta,
            rope_scaling_factor=factor,
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", False)),
            eos_token_ids=eos_ids,
        )
        for name in ("num_hidden_layers", "intermediate_size", "vocab_size", "max_position_embeddings"):
            if getattr(cfg, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(cfg, name)}")
        if cfg.rms_norm_eps <= 0 or cfg.rope_theta <= 0:
            raise ConfigError("rms_norm_eps and rope_theta must be positive")
        return cfg

    def to_json_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "rms_norm_eps": self.rms_norm_eps,
            "vocab_size": self.vocab_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rope_theta": self.rope_theta,
            "tie_word_embeddings": self.tie_word_embeddings,
            "hidden_act": "silu",
            "use_sliding_window": False,
        }
        if self.rope_scaling_factor != 1.0:
            out["rope_scaling"] = {"type": "linear", "factor": self.rope_scaling_factor}
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out


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
