"""Qwen2 / Qwen2.5 dense decoder as a ``ModelSpec``.

What the reference fixes in code rather than reads from ``config.json`` is fixed
here as well, in one place: QKV bias on, O and MLP bias off (``src/decoder_layer.py:28``,
``src/self_attention.py:33``, ``src/mlp.py:9-10``), SiLU (``src/mlp.py:15``), one rotary
encoding shared by every layer (``src/transformer.py:20-25,36``), every layer attending
to all keys.  Checkpoint names are the Hugging Face Qwen2 ones the reference's loader
expects (``src/weight_loader.py:16-22,83-87``).
"""
from __future__ import annotations

from typing import Optional

from ..config.model_config import Qwen2Config
from ..config.registry import register_architecture
from ..parts import LayerSpec, ModelSpec, PartSpec, ScheduleEntry

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
        LayerSpec(prefix=f"model.layers.{i}.", mixer=mixer, feed_forward=ff, mixer_norm=norm, ff_norm=norm, position="rope")
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
        eos_token_ids=eos,
    )


register_architecture("Qwen2ForCausalLM", Qwen2Config.from_dict, qwen2_spec)
