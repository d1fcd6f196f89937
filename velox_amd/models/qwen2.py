"""Qwen2 / Qwen2.5 dense decoder as a ``ModelSpec``.

What the reference fixes in code rather than reads from ``config.json`` is fixed
here as well, in one place: QKV bias on, O and MLP bias off (``src/decoder_layer.py:28``,
``src/self_attention.py:33``, ``src/mlp.py:9-10``), SiLU (``src/mlp.py:15``), one rotary
encoding shared by every layer (``src/transformer.py:20-25,36``), every layer attending
to all keys.  Checkpoint names are the Hugging Face Qwen2 ones the reference's loader
expects (``src/weight_loader.py:16-22,83-87``).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..config.model_config import ConfigError, ModelConfig, require
from ..config.registry import architecture_name, register_architecture
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

@dataclass
class Qwen2Config(ModelConfig):
    """The keys of a Qwen2 / Qwen2.5 ``config.json`` and their defaults, after the reference's ``ModelConfig.from_hf``
    (``src/config.py:6-42``); unlike the reference, keys that change the arithmetic and that the engine does not implement
    are refused instead of ignored (the reference never reads ``use_sliding_window`` or ``hidden_act`` and silently
    ignores non-linear ``rope_scaling``, ``src/rope.py:11-18``)."""

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
        hidden = require(raw, "hidden_size", int)
        heads = require(raw, "num_attention_heads", int)
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
            num_hidden_layers=require(raw, "num_hidden_layers", int),
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=require(raw, "intermediate_size", int),
            rms_norm_eps=eps,
            vocab_size=require(raw, "vocab_size", int),
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



# reference engine/engine.py:23; used only when neither generation_config.json nor config.json names any
DEFAULT_EOS_TOKEN_IDS = (151643, 151645)


def qwen2_spec(config: Qwen2Config, max_position: Optional[int] = None) -> ModelSpec:
    max_position = int(max_position or config.max_position_embeddings)
    norm = PartSpec.of("rmsnorm", hidden_size=config.hidden_size, eps=config.rms_norm_eps)
    mixer = PartSpec.of(
        "attention",
        hidden_size=config.hidden_size,
        num_heads=config.num_attention_heads,
        num_kv_heads=config.num_key_value_heads,
        head_dim=config.head_dim,
        qkv_bias=True,
        window=None,
    )
    ff = PartSpec.of("gated_mlp", hidden_size=config.hidden_size, intermediate_size=config.intermediate_size, activation="silu")
    layers = [
        LayerSpec(prefix=f"model.layers.{i}.", mixer=mixer, feed_forward=ff, mixer_norm=norm, ff_norm=norm, position="rope",
                  mixer_prefix="self_attn.", feed_forward_prefix="mlp.", mixer_norm_prefix="input_layernorm.", ff_norm_prefix="post_attention_layernorm.")
        for i in range(config.num_hidden_layers)
    ]
    eos = tuple(config.eos_token_ids) or tuple(t for t in DEFAULT_EOS_TOKEN_IDS if t < config.vocab_size)
    return ModelSpec(
        vocab_size=config.vocab_size,
        hidden_size=config.hidden_size,
        max_position=max_position,
        layers=layers,
        schedule=[ScheduleEntry(i) for i in range(config.num_hidden_layers)],
        final_norm=norm,
        positions={
            "rope": PartSpec.of(
                "rotary",
                rotary_dim=config.head_dim,
                theta=config.rope_theta,
                max_position=max_position,
                scaling_factor=config.rope_scaling_factor,
            )
        },
        tie_head=config.tie_word_embeddings,
        embed_name="model.embed_tokens.weight",
        head_name="lm_head.weight",
        final_norm_prefix="model.norm.",
        eos_token_ids=eos,
    )


register_architecture("Qwen2ForCausalLM", Qwen2Config.from_dict, qwen2_spec, model_types=("qwen2",))
