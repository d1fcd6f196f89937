from .model_config import ConfigError, ModelConfig, Qwen2Config, read_config_json, read_generation_eos  # noqa: F401
from .registry import (  # noqa: F401
    config_from_dict, get_architecture, known_architectures, load_config, register_architecture,
)
from .engine_config import EngineConfig, resolve_dtype  # noqa: F401
