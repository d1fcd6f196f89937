"""Typed configuration and the architecture registry."""
import json

import pytest

from helpers import TINY_A, TINY_B, TINY_C
from velox_amd.config import ConfigError, config_from_dict, known_architectures, load_config
from velox_amd.models.qwen2 import Qwen2Config
from velox_amd.config.engine_config import EngineConfig, resolve_dtype
from velox_amd.config.registry import get_architecture


def test_reads_every_key_and_defaults():
    cfg = config_from_dict(TINY_B)
    assert isinstance(cfg, Qwen2Config)
    assert (cfg.num_hidden_layers, cfg.hidden_size, cfg.num_attention_heads, cfg.num_key_value_heads) == (3, 96, 3, 1)
    assert cfg.head_dim == 32 and cfg.intermediate_size == 224 and cfg.vocab_size == 320
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5 and not cfg.tie_word_embeddings
    minimal = {"architectures": ["Qwen2ForCausalLM"], "hidden_size": 64, "num_hidden_layers": 1, "num_attention_heads": 4,
               "intermediate_size": 32, "vocab_size": 50}
    cfg = config_from_dict(minimal)
    # defaults of absent keys as the reference's ModelConfig.from_hf has them (src/config.py:34-41)
    assert cfg.num_key_value_heads == 4 and cfg.rms_norm_eps == 1e-6 and cfg.max_position_embeddings == 4096
    assert cfg.rope_theta == 10000.0 and cfg.rope_scaling_factor == 1.0 and cfg.tie_word_embeddings is False
    assert config_from_dict({**minimal, "layer_norm_eps": 1e-3}).rms_norm_eps == 1e-3
    assert config_from_dict({**minimal, "seq_length": 123}).max_position_embeddings == 123


def test_head_dim_key_wins_over_quotient():
    cfg = config_from_dict(TINY_C)
    assert cfg.head_dim == 48 and cfg.hidden_size // cfg.num_attention_heads != 48
    assert cfg.rope_scaling_factor == 2.0


@pytest.mark.parametrize("change,fragment", [
    ({"use_sliding_window": True}, "use_sliding_window"),
    ({"rope_scaling": {"type": "yarn", "factor": 4.0}}, "rope_scaling"),
    ({"hidden_act": "gelu"}, "hidden_act"),
    ({"num_key_value_heads": 3}, "multiple"),
    ({"hidden_size": 66}, "divisible"),
    ({"vocab_size": None}, "vocab_size"),
    ({"architectures": ["LlamaForCausalLM"]}, "unknown architecture"),
    ({"architectures": [], "model_type": None}, "architectures"),
])
def test_refuses_what_it_does_not_implement(change, fragment):
    raw = {**TINY_A, **change}
    with pytest.raises(ConfigError) as err:
        config_from_dict(raw)
    assert fragment in str(err.value)


def test_model_type_stands_in_for_a_missing_class_name():
    raw = {k: v for k, v in TINY_A.items() if k != "architectures"}
    assert config_from_dict(raw).architecture == "Qwen2ForCausalLM"
    with pytest.raises(ConfigError):
        config_from_dict({**raw, "model_type": "other"})


def test_unknown_architecture_lists_known_ones():
    with pytest.raises(ConfigError) as err:
        get_architecture("NopeForCausalLM")
    assert "Qwen2ForCausalLM" in str(err.value) and "Qwen2ForCausalLM" in known_architectures()


def test_round_trip_through_a_folder(tmp_path):
    cfg = config_from_dict(TINY_C)
    (tmp_path / "config.json").write_text(json.dumps(cfg.to_json_dict()))
    again = load_config(str(tmp_path))
    for key in ("hidden_size", "head_dim", "rope_scaling_factor", "rms_norm_eps", "vocab_size", "tie_word_embeddings"):
        assert getattr(again, key) == getattr(cfg, key)
    with pytest.raises(ConfigError):
        load_config(str(tmp_path / "missing"))


def test_spec_has_no_size_of_its_own():
    cfg = config_from_dict(TINY_B)
    spec = get_architecture(cfg.architecture).make_spec(cfg, None)
    assert len(spec.layers) == 3 and len(spec.schedule) == 3 and spec.vocab_size == 320
    mixer = spec.layers[0].mixer.kwargs()
    assert mixer["num_heads"] == 3 and mixer["num_kv_heads"] == 1 and mixer["head_dim"] == 32 and mixer["qkv_bias"] is True
    assert spec.layers[0].feed_forward.kwargs()["intermediate_size"] == 224
    assert spec.final_norm.kwargs()["eps"] == 1e-5
    assert spec.positions["rope"].kwargs()["theta"] == 1e6


def test_engine_config_checks():
    import torch

    assert resolve_dtype("bf16") is torch.bfloat16 and resolve_dtype("float32") is torch.float32 and resolve_dtype("auto") is torch.bfloat16
    with pytest.raises(ValueError):
        resolve_dtype("int8")
    EngineConfig().validate()
    EngineConfig(kv_cache_dtype="auto", quantization=None, download_dir="/nowhere").validate()  # the reference's defaults are accepted
    for bad in (dict(max_num_seqs=0), dict(max_num_batched_tokens=100, max_prefill_chunk_size=512), dict(block_size=12),
                dict(gpu_memory_utilization=0.0), dict(max_num_batched_tokens=16, max_prefill_chunk_size=8, max_num_seqs=32),
                dict(kv_cache_dtype="fp8"), dict(quantization="int8")):
        with pytest.raises(ValueError):
            EngineConfig(**bad).validate()


def test_head_sizes_the_kernels_do_not_take_are_refused_when_the_model_is_built():
    import torch

    from velox_amd.engine.engine import build_model

    for head_dim in (40, 8, 272):
        cfg = config_from_dict({**TINY_A, "head_dim": head_dim})
        with pytest.raises(ValueError) as err:
            build_model(cfg, torch.float32, torch.device("cpu"))
        assert f"head_dim={head_dim}" in str(err.value) and "multiples of 16" in str(err.value)
    build_model(config_from_dict({**TINY_A, "head_dim": 80}), torch.float32, torch.device("cpu"))
