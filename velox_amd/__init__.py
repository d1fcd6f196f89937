"""velox_amd: a single-GPU inference engine for MI355X (gfx950).

Python entry point, in the reference's manner (reference ``README.md:184-194``)::

    from velox_amd import Engine, EngineConfig, Request, SamplingParams
    engine = Engine.from_pretrained(EngineConfig(model="/path/to/model_folder"))
    request = Request("r0", prompt_token_ids=[...], sampling_params=SamplingParams(max_tokens=64))
    engine.generate([request])
    print(request.output_token_ids)
"""
from .config import EngineConfig, load_config  # noqa: F401
from .engine import Engine, Request  # noqa: F401
from .sampling import SamplingParams  # noqa: F401

__all__ = ["Engine", "EngineConfig", "Request", "SamplingParams", "load_config"]
