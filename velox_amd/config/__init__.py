from .model_config import ConfigError, ModelConfig, read_config_json, read_generation_eos, require  # noqa: F401
from .registry import (  # noqa: F401
    architecture_name, config_from_dict, get_architecture, known_architectures, load_config, register_architecture,
)
from .engine_config import EngineConfig, resolve_dtype  # noqa: F401
