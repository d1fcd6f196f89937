"""Random weights from a configuration and a seed.

The reference has no such mode.  The law: every projection, embedding, head and bias
tensor is N(0, 0.02); every norm weight is 1 + N(0, 0.02) (so that a norm applied in
the wrong place changes the result).  Tensors are drawn per CHECKPOINT name, in the
order the model's parts declare them (embedding; per layer: mixer norm, mixer,
feed-forward norm, feed-forward; final norm; head unless tied), each from
``torch.Generator`` seeded with ``seed`` and advanced sequentially, in float32, then
rounded once to the storage dtype.  ``RandomSource`` is such a stream of named tensors
with the face of a checkpoint: ``write_random_model`` stores it as an ordinary model
folder, which the engine then reads like any other, and ``bind_random`` hands it to
the binder that also reads folders (``loader.bind``), for shapes too large to write out.
With the generator on the host both hold the same values; a generator on the device
draws other values of the same law, much faster.
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Iterator, Tuple

import torch
from safetensors.torch import save_file

from ..config.registry import config_from_dict, get_architecture
from ..parts.model import DecoderModel
from .loader import bind, expected_names

_STD = 0.02


def _draw(shape, init: str, generator: torch.Generator, device) -> torch.Tensor:
    values = torch.randn(tuple(shape), generator=generator, dtype=torch.float32, device=device) * _STD
    if init == "one_plus_normal":
        values = values + 1.0
    elif init != "normal":
        raise ValueError(f"unknown init law {init!r}")
    return values


class RandomSource:
    """The tensors a model declares, drawn at random, under their checkpoint names (the binder's ``TensorSource``).
    Values come from ONE generator that advances from tensor to tensor, so they must be asked for in the order of
    declaration; a name that several parameters read is kept until its last reader has had it."""

    def __init__(self, model: DecoderModel, seed: int, storage_dtype: torch.dtype = torch.bfloat16, generator_device: str = "cpu") -> None:
        self.storage_dtype = storage_dtype
        self.device = torch.device(generator_device)
        self.generator = torch.Generator(device=self.device)
        self.generator.manual_seed(int(seed))
        self._law: Dict[str, Tuple[Tuple[int, ...], str]] = {}
        self._readers: Dict[str, int] = {}
        self.order = []
        for _part, _attr, param, names in expected_names(model.all_parts()):
            if param.alias_of is not None:
                continue  # shares another parameter's tensor: nothing of its own is stored
            for name, shape in zip(names, param.source_shapes):
                if name not in self._law:
                    self._law[name] = (tuple(shape), param.init)
                    self.order.append(name)
                self._readers[name] = self._readers.get(name, 0) + 1
        self._next = 0
        self._kept: Dict[str, torch.Tensor] = {}

    def names(self):
        return self._law.keys()

    def __contains__(self, name: str) -> bool:
        return name in self._law

    def shape(self, name: str) -> Tuple[int, ...]:
        return self._law[name][0]

    def tensor(self, name: str) -> torch.Tensor:
        if name in self._kept:
            value = self._kept[name]
        else:
            if self._next >= len(self.order) or self.order[self._next] != name:
                expected = self.order[self._next] if self._next < len(self.order) else "nothing more"
                raise RuntimeError(f"random tensors come from one generator, in order of declaration: asked for {name!r} where {expected!r} is next")
            self._next += 1
            shape, init = self._law[name]
            value = _draw(shape, init, self.generator, self.device).to(self.storage_dtype)
        self._readers[name] -= 1
        if self._readers[name] > 0:
            self._kept[name] = value
        else:
            self._kept.pop(name, None)
        return value


def random_tensors(model: DecoderModel, seed: int, storage_dtype: torch.dtype = torch.float32) -> Iterator[Tuple[str, torch.Tensor]]:
    source = RandomSource(model, seed, storage_dtype)
    for name in list(source.order):
        source._readers[name] = 1
        yield name, source.tensor(name)


def write_random_model(config: Dict[str, Any], out_dir: str, seed: int, dtype: str = "bfloat16") -> str:
    """Writes ``config.json`` and ``model.safetensors`` for the configuration dictionary."""
    storage = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}[dtype]
    typed = config_from_dict(config)
    spec = get_architecture(typed.architecture).make_spec(typed, None)
    model = DecoderModel(spec)
    tensors = {name: value.contiguous() for name, value in random_tensors(model, seed, storage)}
    os.makedirs(out_dir, exist_ok=True)
    save_file(tensors, os.path.join(out_dir, "model.safetensors"), metadata={"format": "pt"})
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as handle:
        json.dump(config, handle, indent=2)
    return out_dir


def bind_random(model: DecoderModel, seed: int, run_dtype: torch.dtype, device, storage_dtype: torch.dtype = torch.bfloat16, generator_device: str = "cpu") -> int:
    """Fills ``model`` with random tensors without a folder: the same binder as for a folder, fed from a ``RandomSource``."""
    return bind(model, RandomSource(model, seed, storage_dtype, generator_device), run_dtype, device)
