"""Random weights from a configuration and a seed.

The reference has no such mode.  The law: every projection, embedding, head and bias
tensor is N(0, 0.02); every norm weight is 1 + N(0, 0.02) (so that a norm applied in
the wrong place changes the result).  Tensors are drawn per CHECKPOINT name, in the
order the model's parts declare them (embedding; per layer: mixer norm, mixer,
feed-forward norm, feed-forward; final norm; head unless tied), each from
``torch.Generator`` seeded with ``seed`` and advanced sequentially, in float32 on the
host, then rounded once to the storage dtype.  ``write_random_model`` stores them as an
ordinary model folder; the engine then reads that folder like any other.
``bind_random`` fills a model in memory without a folder (for large shapes); with
``generator_device="cpu"`` it yields the same values as the folder would.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Iterator, Tuple

import torch
from safetensors.torch import save_file

from ..config.registry import config_from_dict, get_architecture
from ..parts.model import DecoderModel
from .loader import expected_names, held_dtype

_STD = 0.02


def _draw(shape, init: str, generator: torch.Generator, device) -> torch.Tensor:
    values = torch.randn(tuple(shape), generator=generator, dtype=torch.float32, device=device) * _STD
    if init == "one_plus_normal":
        values = values + 1.0
    elif init != "normal":
        raise ValueError(f"unknown init law {init!r}")
    return values


def random_tensors(model: DecoderModel, seed: int) -> Iterator[Tuple[str, torch.Tensor]]:
    generator = torch.Generator(device="cpu")
    generator.manual_seed(int(seed))
    seen = set()
    for part, _attr, param, names in expected_names(model.all_parts()):
        if param.alias_of is not None:
            continue
        for name, shape in zip(names, param.source_shapes):
            if name in seen:
                continue
            seen.add(name)
            yield name, _draw(shape, param.init, generator, "cpu")


def write_random_model(config: Dict[str, Any], out_dir: str, seed: int, dtype: str = "bfloat16") -> str:
    """Writes ``config.json`` and ``model.safetensors`` for the configuration dictionary."""
    storage = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}[dtype]
    typed = config_from_dict(config)
    spec = get_architecture(typed.architecture).make_spec(typed, None)
    model = DecoderModel(spec)
    tensors = {name: value.to(storage).contiguous() for name, value in random_tensors(model, seed)}
    os.makedirs(out_dir, exist_ok=True)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt"})
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(config, handle, indent=2)
    return out_dir


@torch.no_grad()
def bind_random(model: DecoderModel, seed: int, run_dtype: torch.dtype, device, storage_dtype: torch.dtype = torch.bfloat16, generator_device: str = "cpu") -> int:
    device = torch.device(device)
    gen_device = torch.device(generator_device)
    generator = torch.Generator(device=gen_device)
    generator.manual_seed(int(seed))
    bound: Dict[str, torch.Tensor] = {}
    count = 0
    deferred = []
    for part, attr, param, names in expected_names(model.all_parts()):
        if param.alias_of is not None:
            deferred.append((part, attr, param))
            continue
        dtype = held_dtype(param.role, storage_dtype, run_dtype)
        target = torch.empty(param.shape, dtype=dtype, device=device)
        row = 0
        for shape in param.source_shapes:
            piece = _draw(shape, param.init, generator, gen_device).to(storage_dtype)
            n = shape[0]
            target[row:row + n].copy_(piece.to(dtype))
            row += n
        setattr(part, attr, target)
        if len(names) == 1:
            bound[names[0]] = target
        count += target.numel()
    for part, attr, param in deferred:
        setattr(part, attr, bound[param.alias_of])
    for part in model.all_parts():
        part.finalize(device, run_dtype)
    return count
